"""Writes tests/golden/reference_vectors.npz and reference_vectors_e4m3.npz by running the
reference's own Python.

Run in the build container only (the reference tree is not present anywhere else):

    python tests/golden/make_golden.py

What it records, and why these need the reference itself rather than a closed form:

* ``int8_linear`` (reference brokefish/nn/quant.py:281-305) on formula-generated inputs:
  the true-division quantiser and the float64 sum over 256-wide k-chunks are not covered
  by any vector the reference stores (its device tests use x * (1/s) and one chunk).
* ``quantise_weights_int8_bytes`` / ``quantise_activations_int8`` (quant.py:246-278) on
  the same inputs.
* the end-to-end forward of ``BrokefishNet`` (brokefish/nn/model.py:621-645) in fp32 and
  under ``emulated_forward(..., QuantConfig(fmt="int8"))`` (quant.py:498-506) on a net
  whose weights are filled by the formula in :func:`fill_state_dict` (independent of any
  RNG stream) and on eight build-defined positions, plus the layer-0 inputs of the first
  patched matmul, and ``weight_fingerprint`` (brokefish/train/sync.py:34-49) of that net.

* the e4m3 twins (second file): ``fp8_linear`` (quant.py:360-397), ``quantise_activations``
  (:172-188) and ``quantise_weights_bytes`` (:208-224) on the same inputs with the shipped
  constants (q_max 8, 256-deep tiles, 128-row blocks) and once with the module defaults'
  128-deep tiles at q_max 448, and the end-to-end forward under
  ``emulated_forward(net, QuantConfig(weights=True, activations=True, q_max=8, tile_k=256))``.
  torch's fp32 matmul fixes the summation order inside a k-tile, which no closed form gives.

* (third file, ``python tests/golden/make_golden.py layers``) what the reference's own
  ``emulated_forward`` holds **inside** the golden int8 network, for positions 0-1 and layers 0, 3
  and 7: the residual stream entering the layer, and for each of the four patched matmuls the
  operand bytes and activation scales of ``quantise_activations_int8`` on the tensor the patch
  received, and the exact integer accumulators per 256-deep k-chunk of
  ``int8_linear`` (quant.py:299-301: the product of those operands with
  ``quantise_weights_int8_bytes`` of the module's weight) -- in full for position 0 at layer 0,
  as position-weighted row checksums elsewhere; the layer's output for position 0.  And the
  value of the pooled / prenorm value heads (model.py:576-617), 1 and 3 value rows, in fp32 and
  int8-simulated, on the eight positions.

* (fourth file, ``python tests/golden/make_golden.py expand``, reference_vectors_expand.npz) the
  search's expand step as the reference's own ``Search._expand`` performs it
  (brokefish/search/torch_impl.py:962-1033) at E = 96 and E = 16 on the eight positions above and
  the reference's edge-case positions (tests/edge_positions.py), with formula logits: edge moves,
  fp16 priors, edge counts, node values, candidate counts and the truncated prior mass; and on the
  way the position words of ``env.from_fen`` and the legal-move words and check flags of
  ``env.movegen`` (brokefish/env/torch_impl.py:781, :254) for the edge-case positions.

Inputs are regenerated from the formulas below by the tests; only outputs are stored.
"""
from __future__ import annotations

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE = "/root/reference"


def formula(shape, a: int, b: int, mod: int, scale: float) -> torch.Tensor:
    """Deterministic pseudo-random fp32 tensor: ((i*a + b) mod `mod` - mod//2) * scale."""
    n = int(np.prod(shape))
    i = np.arange(n, dtype=np.int64)
    v = ((i * a + b) % mod - mod // 2).astype(np.float32) * np.float32(scale)
    return torch.from_numpy(v.reshape(shape))


def fill_state_dict(sd: dict) -> dict:
    """Overwrite every floating tensor of a state_dict with formula values, distinct per
    tensor and per layer; LayerNorm weights near one, biases small."""
    out = {}
    for k_idx, (name, t) in enumerate(sorted(sd.items())):
        if not torch.is_floating_point(t):
            out[name] = t.clone()
            continue
        fan = t.shape[-1] if t.dim() >= 2 else 1
        if t.dim() == 2:
            v = formula(t.shape, 7919 + 2 * k_idx, 104729 * (k_idx + 1), 2003, 1.0 / (1001.0 * fan ** 0.5) * 1.7)
        elif name.endswith("norm1.weight") or name.endswith("norm2.weight") or name == "norm_f.weight":
            v = 1.0 + formula(t.shape, 31 + k_idx, 17 * k_idx, 211, 0.002)
        else:
            v = formula(t.shape, 131 + k_idx, 29 * k_idx, 401, 0.0005)
        out[name] = v.to(t.dtype)
    return out


# Eight build-defined positions: start, two openings with an en-passant flag and moved
# pieces, captures with dead slots, a promoted queen in pawn slot 3, both sides to move,
# a spread of clocks and repetition counts.
def positions():
    start = [8, 9, 10, 11, 12, 13, 14, 15, 65, 70, 130, 133, 192, 199, 259, 324,
             1072, 1073, 1074, 1075, 1076, 1077, 1078, 1079, 1145, 1150, 1210, 1213, 1272, 1279, 1339, 1404]
    b0 = list(start)
    b1 = list(start); b1[4] = 28 | 0x200                       # e2e4, en-passant flag
    b2 = list(b1); b2[4] = 28; b2[20] = 1024 | 36 | 0x200      # ... e7e5 flagged
    b3 = list(b2); b3[20] = 0x800; b3[9] = 64 | 36; b3[4] = 28  # knight took e5, black pawn dead
    b4 = list(b3); b4[3] = (4 << 6) | 59; b4[30] = 0x800        # promoted queen in pawn slot 3
    b5 = list(b4); b5[15] = 320 | 0x200 | 6; b5[13] = 192 | 5   # white castled short (rook keeps special 0)
    b6 = list(b5); b6[0] = 0x800; b6[1] = 0x800; b6[24] = 0x800; b6[31] = 1024 | 320 | 0x200 | 52
    b7 = list(b6); b7[12] = 192 | 0x200 | 24
    boards = np.array([b0, b1, b2, b3, b4, b5, b6, b7], dtype=np.uint16).view(np.int16)
    control = np.array([1, -1, 1, -1, 37, -101, 100, -2], dtype=np.int16)
    rep = np.array([0, 1, 2, 0, 1, 2, 0, 5], dtype=np.uint8)
    return torch.from_numpy(boards), torch.from_numpy(control), torch.from_numpy(rep)


def weight_checksum(q: np.ndarray) -> np.ndarray:
    """Position-weighted int64 checksums of an int8 matrix (rows and columns)."""
    q = q.astype(np.int64)
    w = np.arange(q.size, dtype=np.int64).reshape(q.shape) % 1009 + 1
    return np.array([(q * w).sum(), q.sum(), np.abs(q).sum(), (q[::3] * w[::3]).sum()], dtype=np.int64)


def linear_cases():
    """(name, x, w, bias, unsigned) for the standalone int8_linear vectors."""
    cases = []
    x1 = formula((32, 256), 31, 7, 401, 0.004) * (1.0 + 0.05 * torch.arange(32)[:, None])
    w1 = formula((256, 256), 11, 5, 255, 0.0007)
    cases.append(("s8_k256", x1, w1, formula((256,), 3, 1, 101, 0.01), False))
    x2 = torch.relu(formula((32, 1024), 17, 3, 409, 0.003) * (1.0 + 0.03 * torch.arange(32)[:, None]))
    w2 = formula((128, 1024), 13, 9, 251, 0.0009)
    cases.append(("u8_k1024", x2, w2, formula((128,), 5, 2, 103, 0.02), True))
    x3 = formula((16, 512), 29, 11, 397, 0.002)
    w3 = formula((128, 512), 19, 4, 253, 0.0011)
    cases.append(("s8_k512_nobias", x3, w3, None, False))
    x4 = x1.clone(); x4[3] = 0.0                          # an all-zero row: scale must be 1
    cases.append(("s8_zero_row", x4, w1, None, False))
    return cases


def main() -> int:
    sys.path.insert(0, REFERENCE)
    from brokefish.nn import quant as rq                      # noqa: E402
    from brokefish.nn.model import BrokefishNet as RefNet     # noqa: E402

    out = {}
    f8 = {}
    shipped = rq.QuantConfig(weights=True, activations=True, q_max=rq.Q_MAX, tile_k=rq.ROW_K, block_n=rq.BLOCK_N)
    wide = rq.QuantConfig(weights=True, activations=True, q_max=448.0)      # module defaults: 128-deep tiles
    for name, x, w, bias, unsigned in linear_cases():
        f8[f"lin_{name}"] = rq.fp8_linear(x, w, bias, shipped).numpy()
        f8[f"lin128_{name}"] = rq.fp8_linear(x, w, bias, wide).numpy()
        qb, ws = rq.quantise_weights_bytes(w, rq.Q_MAX, tile_k=rq.ROW_K)
        f8[f"wqsum_{name}"] = weight_checksum(qb.numpy())
        f8[f"ws_{name}"] = ws.numpy()
        q, s = rq.quantise_activations(x[:, :256].contiguous(), rq.Q_MAX, rq.ROW_K)
        f8[f"qa_{name}"] = q.to(rq.E4M3).view(torch.uint8).numpy()
        f8[f"sa_{name}"] = s.numpy()
        y = rq.int8_linear(x, w, bias, unsigned=unsigned)
        out[f"lin_{name}"] = y.numpy()
        qb, ws = rq.quantise_weights_int8_bytes(w)
        out[f"wqsum_{name}"] = weight_checksum(qb.view(torch.int8).numpy())
        out[f"ws_{name}"] = ws.numpy()
        q, s = rq.quantise_activations_int8(x[:, :256], unsigned)
        out[f"qa_{name}"] = q.numpy().astype(np.int16)
        out[f"sa_{name}"] = s.numpy()

    for n_value in (1, 3):
        torch.manual_seed(0)
        net = RefNet(n_value=n_value).eval()
        net.load_state_dict(fill_state_dict(net.state_dict()))
        boards, control, rep = positions()
        if n_value == 3:            # the second net only adds the value-head variant
            boards, control, rep = boards[:3], control[:3], rep[:3]
        captured = []
        handle = net.encoder.layers[0].norm1.register_forward_hook(lambda m, i, o: captured.append(o.detach().clone()))
        with torch.no_grad():
            p32, q32, v32 = net(boards, control, rep)
            handle.remove()
            p8, q8, v8 = rq.emulated_forward(net, rq.QuantConfig(fmt="int8"))(boards, control, rep)
            if n_value == 1:
                pf, qf, vf = rq.emulated_forward(net, shipped)(boards, control, rep)
                f8["e4m3_policy_nv1"], f8["e4m3_promo_nv1"], f8["e4m3_value_nv1"] = pf.numpy(), qf.numpy(), vf.numpy()
        tag = f"nv{n_value}"
        out[f"fp32_policy_{tag}"], out[f"fp32_promo_{tag}"], out[f"fp32_value_{tag}"] = p32.numpy(), q32.numpy(), v32.numpy()
        out[f"int8_policy_{tag}"], out[f"int8_promo_{tag}"], out[f"int8_value_{tag}"] = p8.numpy(), q8.numpy(), v8.numpy()
        if n_value == 1:
            out["ln1_layer0"] = captured[0][:2].numpy()        # input of the first patched matmul, boards 0-1
            # the module file alone: its package's __init__ needs a logging library that is not installed
            import importlib.util
            spec = importlib.util.spec_from_file_location("ref_sync", os.path.join(REFERENCE, "brokefish", "train", "sync.py"))
            ref_sync = importlib.util.module_from_spec(spec)
            sys.modules["ref_sync"] = ref_sync                 # its dataclass looks its module up by name
            spec.loader.exec_module(ref_sync)
            out["weight_fingerprint_nv1"] = np.array(ref_sync.weight_fingerprint(net), np.float64)
    out["torch_version"] = np.array(torch.__version__)
    path = os.path.join(HERE, "reference_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, {k: getattr(v, "shape", None) for k, v in out.items()})
    f8["torch_version"] = np.array(torch.__version__)
    path = os.path.join(HERE, "reference_vectors_e4m3.npz")
    np.savez_compressed(path, **f8)
    print("wrote", path, {k: getattr(v, "shape", None) for k, v in f8.items()})
    return 0


LAYER_TAPS = (0, 3, 7)
MATMUL_OF = {"qkv": "self_attn.in_proj_weight", "out": "self_attn.out_proj.weight",
             "ff1": "linear1.weight", "ff2": "linear2.weight"}


def row_checksum(acc: np.ndarray) -> np.ndarray:
    """[..., N] integer accumulators -> [...] int64: sum over the output channel n of acc * (n % 1009 + 1)."""
    w = (np.arange(acc.shape[-1], dtype=np.int64) % 1009) + 1
    return (acc.astype(np.int64) * w).sum(axis=-1)


def main_layers() -> int:
    sys.path.insert(0, REFERENCE)
    from brokefish.nn import quant as rq                      # noqa: E402
    from brokefish.nn.model import BrokefishNet as RefNet     # noqa: E402

    out = {}
    torch.manual_seed(0)
    net = RefNet(n_value=1).eval()
    net.load_state_dict(fill_state_dict(net.state_dict()))
    boards, control, rep = positions()
    boards, control, rep = boards[:2], control[:2], rep[:2]
    which = {}
    for l in LAYER_TAPS:
        lay = net.encoder.layers[l]
        which[id(lay.self_attn.in_proj_weight)] = (l, "qkv")
        which[id(lay.self_attn.out_proj.weight)] = (l, "out")
        which[id(lay.linear1.weight)] = (l, "ff1")
        which[id(lay.linear2.weight)] = (l, "ff2")
    original = rq.int8_linear

    def recording(x, w, bias, unsigned=False, row_k=rq.ROW_K):
        tag = which.get(id(w))
        if tag is not None:
            l, name = tag
            a = x.reshape(-1, x.shape[-1]).float()
            wq, ws = rq.quantise_weights_int8_bytes(w.float())
            wq = wq.view(torch.int8).double()
            qs, sas, accs = [], [], []
            for lo in range(0, a.shape[1], row_k):
                tq, sa = rq.quantise_activations_int8(a[:, lo:lo + row_k], unsigned)
                qs.append(tq)
                sas.append(sa)
                accs.append((tq.double() @ wq[:, lo:lo + row_k].T).round().to(torch.int64))
            # rows arrive as (position, token) outside the attention module and as (token, position)
            # inside it (torch's multi_head_attention_forward works on [T, B, E])
            inside = name in ("qkv", "out")

            def by_position(t):      # [rows, C] -> [2, 32, C]
                return t.reshape(32, 2, -1).transpose(0, 1) if inside else t.reshape(2, 32, -1)

            q = by_position(torch.cat(qs, dim=1))
            acc = torch.stack([by_position(a_) for a_ in accs]).numpy()            # [kc, 2, 32, N]
            assert np.abs(acc).max() < 2 ** 31
            key = f"l{l}_{name}"
            out[f"qa_{key}"] = q.numpy().astype(np.uint8 if unsigned else np.int8)
            out[f"sa_{key}"] = by_position(torch.cat(sas, dim=1)).numpy()
            out[f"accsum_{key}"] = row_checksum(acc)                              # [kc, 2, 32]
            if l == LAYER_TAPS[0]:
                out[f"acc_{key}"] = acc[:, 0].astype(np.int32)                    # position 0 in full
        return original(x, w, bias, unsigned=unsigned, row_k=row_k)

    hooks = []
    for l in LAYER_TAPS:
        hooks.append(net.encoder.layers[l].register_forward_pre_hook(
            lambda m, args, l=l: out.__setitem__(f"x_in_l{l}", args[0].detach().clone().numpy())))
        hooks.append(net.encoder.layers[l].register_forward_hook(
            lambda m, args, o, l=l: out.__setitem__(f"x_out_l{l}", o.detach()[:1].clone().numpy())))
    rq.int8_linear = recording
    try:
        with torch.no_grad():
            p8, q8, v8 = rq.emulated_forward(net, rq.QuantConfig(fmt="int8"))(boards, control, rep)
    finally:
        rq.int8_linear = original
        for h in hooks:
            h.remove()
    out["int8_policy_2"], out["int8_value_2"] = p8.numpy(), v8.numpy()

    # the pooled value heads: same formula weights (the marker buffer is not a float tensor and
    # sorts after every float key), so policy and promotion logits are those of the king net
    boards, control, rep = positions()
    for head in ("pooled", "prenorm"):
        for n_value in (1, 3):
            torch.manual_seed(0)
            vnet = RefNet(n_value=n_value, value_head=head).eval()
            vnet.load_state_dict(fill_state_dict(vnet.state_dict()))
            with torch.no_grad():
                p32, q32, v32 = vnet(boards, control, rep)
                p8, q8, v8 = rq.emulated_forward(vnet, rq.QuantConfig(fmt="int8"))(boards, control, rep)
            out[f"fp32_value_{head}_nv{n_value}"], out[f"int8_value_{head}_nv{n_value}"] = v32.numpy(), v8.numpy()
            out[f"int8_policysum_{head}_nv{n_value}"] = np.array(p8.double().sum().item())
    out["torch_version"] = np.array(torch.__version__)
    path = os.path.join(HERE, "reference_vectors_layers.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, {k: getattr(v, "shape", None) for k, v in out.items()}, os.path.getsize(path), "bytes")
    return 0


def expand_logits(n: int):
    """Formula logits for the expand vectors: policy [n,32,64], promo [n,32,4], value [n] in (-1, 1)."""
    policy = formula((n, 32, 64), 7907, 13, 4001, 0.0015)
    promo = formula((n, 32, 4), 6101, 5, 811, 0.004)
    value = formula((n,), 397, 3, 199, 0.0099)
    return policy, promo, value


def main_expand() -> int:
    sys.path.insert(0, REFERENCE)
    sys.path.insert(0, os.path.dirname(HERE))                       # tests/: the list of edge-case FENs
    sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))      # the repository root
    from brokefish.env import torch_impl as env
    from brokefish.search.torch_impl import Search, SearchConfig
    import edge_positions as ep

    fb, fc = zip(*(env.from_fen(f) for _, f in ep.ALL))
    fen_boards, fen_control = torch.cat(fb), torch.cat(fc)
    gb, gc, _ = positions()
    boards = torch.cat([gb, fen_boards.to(torch.int16)])
    control = torch.cat([gc, fen_control.to(torch.int16)])
    n = boards.shape[0]
    mask, in_check = env.movegen(boards, control)
    policy, promo, value = expand_logits(n)
    out = {"fen_boards": fen_boards.to(torch.int16).numpy(), "fen_control": fen_control.to(torch.int16).numpy(),
           "mask": mask.numpy(), "in_check": in_check.numpy()}
    for E in (96, 16):
        s = Search(SearchConfig(n=1, B=n, E=E), evaluate=None, device="cpu", check_invariants=False)
        s.node_board[:, 0] = boards
        s.node_control[:, 0] = control
        rec = {}
        s.stats.on_expand = lambda count, n_edges, dropped, do: rec.update(count=count.clone(), dropped=dropped.clone())
        s._expand(torch.zeros(n, dtype=torch.long), mask, torch.ones(n, dtype=torch.bool), policy, promo, value)
        out[f"edge_move_E{E}"] = s.edge_move[:, 0].numpy().copy()
        out[f"edge_prior_E{E}"] = s.edge_prior[:, 0].numpy().copy()
        out[f"n_edges_E{E}"] = s.node_nedges[:, 0].numpy().copy()
        out[f"node_value_E{E}"] = s.node_value[:, 0].numpy().copy()
        out[f"count_E{E}"] = rec["count"].numpy().astype(np.int32)
        out[f"dropped_E{E}"] = rec["dropped"].numpy().astype(np.float32)
    path = os.path.join(HERE, "reference_vectors_expand.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {os.path.getsize(path)} bytes, {n} positions, counts {out['count_E96'].tolist()}")
    return 0


if __name__ == "__main__":
    mode = sys.argv[1:]
    raise SystemExit(main_layers() if mode == ["layers"] else main_expand() if mode == ["expand"] else main())
