"""Shared by the CPU and GPU tests that hold an implementation to the per-layer data the reference's
own ``emulated_forward`` wrote (tests/golden/reference_vectors_layers.npz, made by
tests/golden/make_golden.py from brokefish/nn/quant.py:246-305 and :443-506).

For positions 0-1 and layers 0, 3, 7 of the golden int8 network the fixture holds the residual
stream entering the layer and, for each of the four matmuls, the reference's operand bytes,
activation scales and int32 accumulators.  An implementation is run on ONE layer from the
reference's residual stream and must then reproduce

* the reference's operand bytes -- except where the quotient x / s, recomputed here in float64
  from the reference's own upstream bytes, lies within ``TIE_TOL`` of a rounding boundary k + 1/2
  (there two fp32 summation orders may legitimately round to different sides);
* the reference's accumulators, exactly, wherever the operand rows are identical (integer
  arithmetic has no tolerance);

A position's chain of stages is followed until the first stage with a tie flip (a flipped byte
changes everything downstream of it, so later stages of that chain are no longer comparable).
"""
import math
import os

import numpy as np
import torch

import make_golden as mg
from brokefish_amd import hip_impl
from brokefish_amd.net import BrokefishNet

LAYERS = mg.LAYER_TAPS
# distance of a quotient from k + 1/2, in quantisation steps, below which a different rounding is
# accepted: 2^-18 of the full scale of 127 steps (fp32 re-ordering noise of a LayerNorm or
# attention output is about 2^-21 of the row's largest value)
TIE_TOL = 127.0 * 2.0 ** -18
TIE_TOL_U8 = 255.0 * 2.0 ** -18      # the unsigned quantiser of the second feed-forward matmul


def tie_distance(q64):
    """distance of each quotient from the nearest k + 1/2, in quantisation steps"""
    q64 = np.asarray(q64, dtype=np.float64)
    return np.abs(q64 - (np.floor(q64) + 0.5))


def _e4m3_grid():
    """the non-negative finite values of OCP e4m3 (4 exponent bits, bias 7, 3 mantissa bits, max 448)"""
    v = [m / 8.0 * 2.0 ** -6 for m in range(8)]
    v += [(1 + m / 8.0) * 2.0 ** (e - 7) for e in range(1, 16) for m in range(8)]
    return np.array(sorted(x for x in v if x <= 448.0))


E4M3_GRID = _e4m3_grid()
# distance of a quotient from the midpoint of two neighbouring e4m3 values below which a different
# rounding is accepted: 2^-18 of the full scale (a row's largest magnitude is mapped to 8).  Measured
# on MI355X: flipped bytes sit within 7e-8 of a midpoint at a layer's first quantiser (identical
# input up to a LayerNorm's fp32 summation order) and within 4e-7 behind a matmul (whose fp32 sum
# over 256 products differs between two orderings by about 2^-24 of sum|a*w|).
E4M3_TIE_TOL = 8.0 * 2.0 ** -18
E4M3_TIE_TOL_AFTER_MATMUL = 8.0 * 2.0 ** -18


def e4m3_tie_distance(q64):
    """absolute distance of each quotient from the nearest midpoint of two neighbouring e4m3 values"""
    a = np.minimum(np.abs(np.asarray(q64, dtype=np.float64)), 448.0)
    hi = np.clip(np.searchsorted(E4M3_GRID, a, side="right"), 1, len(E4M3_GRID) - 1)
    mid = 0.5 * (E4M3_GRID[hi - 1] + E4M3_GRID[hi])
    # the midpoint below the lower neighbour can be the nearer one
    lo = np.clip(hi - 1, 1, None)
    mid_below = 0.5 * (E4M3_GRID[lo - 1] + E4M3_GRID[lo])
    return np.minimum(np.abs(a - mid), np.abs(a - mid_below))


def load():
    fx = np.load(os.path.join(os.path.dirname(mg.__file__), "reference_vectors_layers.npz"))
    torch.manual_seed(0)
    net = BrokefishNet(n_value=1).eval()
    sd = mg.fill_state_dict(net.state_dict())
    net.load_state_dict(sd)
    b, c, r = mg.positions()
    return fx, net, sd, b[:2], c[:2], r[:2]


def _weights(sd, l):
    p = f"encoder.layers.{l}."
    out = {}
    for name, key, bias in (("qkv", "self_attn.in_proj_weight", "self_attn.in_proj_bias"),
                            ("out", "self_attn.out_proj.weight", "self_attn.out_proj.bias"),
                            ("ff1", "linear1.weight", "linear1.bias"), ("ff2", "linear2.weight", "linear2.bias")):
        q, s = hip_impl.quantise_weights_int8(sd[p + key])
        out[name] = (q.astype(np.int64), s, sd[p + bias].numpy())
    return out


def _linear_fp32(qa, sa, wq, ws, bias):
    """The reference's int8_linear from given operand bytes: exact integer products per 256-deep
    chunk, float64 sum of acc * sa, one cast, fp32 * ws, fp32 + bias (quant.py:296-304)."""
    k = qa.shape[1]
    out64 = np.zeros((qa.shape[0], wq.shape[0]), np.float64)
    accs = []
    for ci, lo in enumerate(range(0, k, 256)):
        acc = qa[:, lo:lo + 256].astype(np.int64) @ wq[:, lo:lo + 256].T
        accs.append(acc)
        out64 += acc.astype(np.float64) * sa[:, ci:ci + 1].astype(np.float64)
    out = out64.astype(np.float32) * np.repeat(ws, 128)[None, :].astype(np.float32)
    return (out + bias.astype(np.float32)).astype(np.float32), np.stack(accs)


def _ln64(x, g, b, eps=1e-5):
    x = x.astype(np.float64)
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * g.astype(np.float64) + b.astype(np.float64)


def reference_stages(fx, sd, l, pos, alive):
    """float64 quotients entering each of the four quantisers of layer ``l`` for position ``pos``,
    recomputed from the reference's own upstream bytes, plus the reference's bytes / accumulators."""
    p = f"encoder.layers.{l}."
    w = _weights(sd, l)
    x_in = fx[f"x_in_l{l}"][pos]
    st = {}
    y64 = _ln64(x_in, sd[p + "norm1.weight"].numpy(), sd[p + "norm1.bias"].numpy())
    st["qkv"] = y64 / fx[f"sa_l{l}_qkv"][pos].astype(np.float64)
    qkv, acc_qkv = _linear_fp32(fx[f"qa_l{l}_qkv"][pos], fx[f"sa_l{l}_qkv"][pos], *w["qkv"])
    d = 256
    q, k, v = (qkv[:, i * d:(i + 1) * d].astype(np.float64).reshape(32, 8, 32).transpose(1, 0, 2) for i in range(3))
    s = q @ k.transpose(0, 2, 1) / math.sqrt(32.0)
    s[:, :, ~alive] = -np.inf
    pr = np.exp(s - s.max(-1, keepdims=True))
    pr /= pr.sum(-1, keepdims=True)
    o64 = (pr @ v).transpose(1, 0, 2).reshape(32, d)
    st["out"] = o64 / fx[f"sa_l{l}_out"][pos].astype(np.float64)
    att, acc_out = _linear_fp32(fx[f"qa_l{l}_out"][pos], fx[f"sa_l{l}_out"][pos], *w["out"])
    x_mid = (x_in + att).astype(np.float32)
    y64 = _ln64(x_mid, sd[p + "norm2.weight"].numpy(), sd[p + "norm2.bias"].numpy())
    st["ff1"] = y64 / fx[f"sa_l{l}_ff1"][pos].astype(np.float64)
    hid, acc_ff1 = _linear_fp32(fx[f"qa_l{l}_ff1"][pos], fx[f"sa_l{l}_ff1"][pos], *w["ff1"])
    hid = np.maximum(hid, np.float32(0))
    st["ff2"] = hid.astype(np.float64) / np.repeat(fx[f"sa_l{l}_ff2"][pos].astype(np.float64), 256, axis=1)
    ff, acc_ff2 = _linear_fp32(fx[f"qa_l{l}_ff2"][pos], fx[f"sa_l{l}_ff2"][pos], *w["ff2"])
    x_out = (x_mid + ff).astype(np.float32)
    accs = {"qkv": acc_qkv, "out": acc_out, "ff1": acc_ff1, "ff2": acc_ff2}
    # the fixture's accumulators are these integer products: the reference computed them from the
    # same operands (full for position 0 at the first tapped layer, row checksums everywhere)
    for name, a in accs.items():
        assert (mg.row_checksum(a) == fx[f"accsum_l{l}_{name}"][:, pos]).all(), (l, pos, name)
        if pos == 0 and l == LAYERS[0]:
            assert (a == fx[f"acc_l{l}_{name}"]).all(), (l, name)
    return st, accs, x_out


def check(run_layer, report=None):
    """``run_layer(l, x_in [2,32,256] fp32) -> dict`` of numpy taps for that one layer (qa_* [2,1,32,K],
    acc_* [2,1,kc,32,N], resid [2,1,32,256]).  Returns the statistics it asserted on."""
    fx, net, sd, b, c, r = load()
    alive_all = ((b.numpy().view(np.uint16) >> 11) & 1) == 0
    stats = {"chains": 0, "clean_chains": 0, "stages_checked": 0, "tie_flips": 0, "bytes_compared": 0,
             "worst_tie_distance": 0.0, "worst_resid_error": 0.0}
    for l in LAYERS:
        got = run_layer(l, fx[f"x_in_l{l}"])
        for pos in range(2):
            st, accs, x_out = reference_stages(fx, sd, l, pos, alive_all[pos])
            stats["chains"] += 1
            clean = True
            for name in ("qkv", "out", "ff1", "ff2"):
                ref_q = fx[f"qa_l{l}_{name}"][pos].astype(np.int64)
                got_q = got[f"qa_{name}"][pos, 0].astype(np.int64)
                if name == "ff2":
                    got_q = got[f"qa_{name}"][pos, 0].view(np.uint8).astype(np.int64)
                diff = got_q != ref_q
                stats["bytes_compared"] += diff.size
                stats["stages_checked"] += 1
                if diff.any():
                    assert (np.abs(got_q - ref_q)[diff] == 1).all(), (l, pos, name, "a flipped byte must be the neighbouring value")
                    dist = tie_distance(st[name])[diff]
                    tol = TIE_TOL_U8 if name == "ff2" else TIE_TOL
                    stats["worst_tie_distance"] = max(stats["worst_tie_distance"], float(dist.max()))
                    assert (dist <= tol).all(), \
                        f"layer {l} position {pos} matmul {name}: {int(diff.sum())} bytes differ from the reference's and " \
                        f"the worst sits {dist.max():.3g} steps from a rounding boundary (allowed {tol:.3g})"
                    stats["tie_flips"] += int(diff.sum())
                    clean = False
                # accumulators: exact on every row whose operand bytes are the reference's
                rows = ~diff.any(axis=1)
                got_acc = got[f"acc_{name}"][pos, 0].astype(np.int64)            # [kc, 32, N]
                assert (got_acc[:, rows] == accs[name][:, rows]).all(), (l, pos, name, "int32 accumulators")
                if not clean:
                    break
            if clean:
                stats["clean_chains"] += 1
                err = float(np.abs(got["resid"][pos, 0] - x_out).max() / max(1.0, np.abs(x_out).max()))
                stats["worst_resid_error"] = max(stats["worst_resid_error"], err)
                assert err < 2e-5, (l, pos, err)
                if pos == 0:   # the layer output the reference itself produced
                    assert np.abs(got["resid"][0, 0] - fx[f"x_out_l{l}"][0]).max() < 2e-5 * max(1.0, np.abs(x_out).max())
    assert stats["clean_chains"] >= 3, stats
    if report is not None:
        report(stats)
    return stats
