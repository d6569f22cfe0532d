"""TEST INFRASTRUCTURE -- NOT PRODUCT CODE.

A CPU restatement, in plain PyTorch library calls, of the reference network forward in
its modes: fp32, the int8-simulated forward the HIP evaluator must reproduce, and the
e4m3-simulated forward of its fp8 variant.
Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU-baseline leg import
this module; nothing under ``brokefish_amd/`` does.

It works on a bare ``state_dict`` (same key names as the reference model,
brokefish/nn/model.py:297-316), so it does not depend on any model class.

What each function follows (paths inside the reference tree):

* :func:`decode_words`, :func:`embed_indices`  -- brokefish/nn/model.py:251-265, :455-477
* :func:`embed`                                 -- brokefish/nn/model.py:635-640 (order normative,
  docs/reference/spec.md:386-391)
* :func:`quantise_activations_int8`             -- brokefish/nn/quant.py:246-260
* :func:`quantise_weights_int8`                 -- brokefish/nn/quant.py:263-278
* :func:`int8_linear`                           -- brokefish/nn/quant.py:281-305
* :func:`quantise_activations_e4m3`, :func:`quantise_weights_e4m3`, :func:`fp8_linear`
                                                -- brokefish/nn/quant.py:161-224, :360-397 with the
  shipped constants q_max = 8 (:105), tile_k = 256 (:92), block_n = 128 (:82), fp32 accumulator
* :func:`forward` block structure               -- torch ``TransformerEncoderLayer(norm_first=True)``
  as constructed at brokefish/nn/model.py:303-311 and called at :525 with
  ``src_key_padding_mask=~alive``; the four matmuls routed through ``int8_linear`` and
  ``ffn2`` unsigned as in brokefish/nn/quant.py:421-440, :466-473
* heads                                         -- brokefish/nn/model.py:551-617
* mask AND / argmax (not in the reference evaluator; the search applies it)
                                                -- docs/reference/spec.md:141-143, :537-540

LayerNorm, softmax and the fp32 matmuls are torch library routines here, so their
summation order is torch's; the C checker ``bf_oracle.c`` fixes explicit orders instead.
The two agree to rounding noise, which ``tests/test_oracle.py`` asserts.
"""
from __future__ import annotations

import contextlib
import math
from typing import Dict, Optional

import torch
import torch.nn.functional as F

ROW_K = 256      # brokefish/nn/quant.py:92
BLOCK_N = 128    # brokefish/nn/quant.py:82
Q_MAX_S8 = 127.0  # brokefish/nn/quant.py:237
Q_MAX_U8 = 255.0  # brokefish/nn/quant.py:241
Q_MAX_E4M3 = 8.0  # brokefish/nn/quant.py:105
E4M3_MAX = 448.0  # brokefish/nn/quant.py:73
E4M3 = torch.float8_e4m3fn   # OCP e4m3: no infinities, maximum 448 (brokefish/nn/quant.py:69-73)
KING_WHITE, KING_BLACK = 15, 31


def decode_words(boards: torch.Tensor):
    w = boards.to(torch.int64) & 0xFFFF
    return (w >> 11) & 1, (w >> 10) & 1, (w >> 9) & 1, (w >> 6) & 7, w & 63


def embed_indices(boards, control, rep):
    captured, colour, special, ptype, square = decode_words(boards)
    stm = (control < 0).to(torch.int64)
    clock = (control.to(torch.int64).abs() - 1).clamp(0, 100)
    return (square, ptype * 2 + special, colour * 2 + stm[:, None], clock,
            rep.to(torch.int64).clamp(0, 2)), captured == 0


def embed(sd: Dict[str, torch.Tensor], boards, control, rep):
    idx, alive = embed_indices(boards, control, rep)
    per_board = sd["emb_clock.weight"][idx[3]] + sd["emb_rep.weight"][idx[4]]
    x = sd["emb_square.weight"][idx[0]]
    x = x + sd["emb_type_special.weight"][idx[1]]
    x = x + sd["emb_color_turn.weight"][idx[2]]
    x = x + per_board[:, None, :]
    return x, alive


def quantise_activations_int8(x: torch.Tensor, unsigned: bool = False):
    """[M, K] fp32 -> (integer-valued fp32 [M, K], scale [M, 1])."""
    if unsigned:
        pos = x.clamp(min=0)
        amax = pos.amax(dim=-1, keepdim=True)
        s = torch.where(amax > 0, amax / Q_MAX_U8, torch.ones_like(amax))
        return torch.round(pos / s).clamp(0, Q_MAX_U8), s
    amax = x.abs().amax(dim=-1, keepdim=True)
    s = torch.where(amax > 0, amax / Q_MAX_S8, torch.ones_like(amax))
    return torch.round(x / s).clamp(-Q_MAX_S8, Q_MAX_S8), s


def quantise_weights_int8(w: torch.Tensor):
    """[N, K] fp32 -> (int8 [N, K], scale [N // 128]); one scale per 128 output rows."""
    n, k = w.shape
    if n % BLOCK_N:
        raise ValueError(f"weight {tuple(w.shape)} does not tile into {BLOCK_N} rows")
    blocks = w.float().reshape(n // BLOCK_N, BLOCK_N * k)
    amax = blocks.abs().amax(dim=1, keepdim=True)
    s = torch.where(amax > 0, amax / Q_MAX_S8, torch.ones_like(amax))
    q = torch.round(blocks / s).clamp(-Q_MAX_S8, Q_MAX_S8).to(torch.int8)
    return q.reshape(n, k), s.reshape(-1).contiguous()


def int8_linear(x, w, bias, unsigned: bool = False, taps: Optional[dict] = None, name: str = ""):
    """``F.linear`` with both operands int8, exact integer accumulation per 256-wide
    k-chunk, float64 across chunks, one weight descale at the end."""
    lead = x.shape[:-1]
    a = x.reshape(-1, x.shape[-1]).float()
    m, k = a.shape
    n = w.shape[0]
    wq, ws = quantise_weights_int8(w)
    wq64 = wq.to(torch.float64)
    out = torch.zeros(m, n, dtype=torch.float64)
    qs, accs, quots = [], [], []
    for lo in range(0, k, ROW_K):
        q, sa = quantise_activations_int8(a[:, lo:lo + ROW_K], unsigned)
        acc = q.to(torch.float64) @ wq64[:, lo:lo + ROW_K].T
        out += acc * sa.to(torch.float64)
        if taps is not None:
            qs.append(q.to(torch.int16))
            accs.append(acc.to(torch.int32))
            src = a[:, lo:lo + ROW_K].clamp(min=0) if unsigned else a[:, lo:lo + ROW_K]
            quots.append(src.to(torch.float64) / sa.to(torch.float64))
    if taps is not None:
        taps.setdefault("qa_" + name, []).append(torch.cat(qs, dim=1))
        taps.setdefault("acc_" + name, []).append(torch.stack(accs))
        # the quotients x / s before rounding, in float64: how far each byte was from a tie
        taps.setdefault("quot_" + name, []).append(torch.cat(quots, dim=1))
    y = out.to(torch.float32) * ws.repeat_interleave(BLOCK_N)[None, :]
    if bias is not None:
        y = y + bias.float()
    return y.reshape(*lead, n)


def _to_e4m3(x: torch.Tensor) -> torch.Tensor:
    """Round to e4m3 and back to fp32; clamped first because the format has no infinity."""
    return x.clamp(-E4M3_MAX, E4M3_MAX).to(E4M3).to(torch.float32)


def quantise_activations_e4m3(x: torch.Tensor, q_max: float = Q_MAX_E4M3, tile_k: int = ROW_K):
    """[M, K] fp32 -> (e4m3-valued fp32 [M, K], scale [M, K // tile_k]); one scale per row
    per k-tile, the tile's largest magnitude landing on ``q_max``."""
    m, k = x.shape
    if k % tile_k:
        raise ValueError(f"K = {k} is not a multiple of the {tile_k}-element tile")
    tiles = x.view(m, k // tile_k, tile_k)
    amax = tiles.abs().amax(dim=-1, keepdim=True)
    s = torch.where(amax > 0, amax / q_max, torch.ones_like(amax))
    return _to_e4m3(tiles / s).view(m, k), s.squeeze(-1)


def quantise_weights_e4m3(w: torch.Tensor, q_max: float = Q_MAX_E4M3, tile_k: int = ROW_K,
                          block_n: int = BLOCK_N):
    """[N, K] fp32 -> (e4m3-valued fp32 [N, K], scale [N // block_n, K // tile_k])."""
    n, k = w.shape
    if n % block_n or k % tile_k:
        raise ValueError(f"weight {tuple(w.shape)} does not tile into {block_n}x{tile_k} blocks")
    blocks = w.view(n // block_n, block_n, k // tile_k, tile_k)
    amax = blocks.abs().amax(dim=(1, 3), keepdim=True)
    s = torch.where(amax > 0, amax / q_max, torch.ones_like(amax))
    return _to_e4m3(blocks / s).view(n, k), s.reshape(n // block_n, k // tile_k)


# How the product inside one k-tile is summed: False = torch's fp32 matmul (the reference's
# call, summation order left to the library), True = exact sum rounded once to fp32 (float64
# holds every partial sum of 256 e4m3 products exactly).  Both are fp32 realisations of the same
# formula; tests use the second to show what a change of summation order alone does.
TILE_SUM_EXACT = False


@contextlib.contextmanager
def exact_tile_sums():
    global TILE_SUM_EXACT
    old, TILE_SUM_EXACT = TILE_SUM_EXACT, True
    try:
        yield
    finally:
        TILE_SUM_EXACT = old


def fp8_linear(x, w, bias, taps: Optional[dict] = None, name: str = "", q_max: float = Q_MAX_E4M3,
               tile_k: int = ROW_K, block_n: int = BLOCK_N):
    """``F.linear`` with both operands e4m3: the product inside one k-tile in fp32, one
    descale ``* sa * sw`` per tile, fp32 sum over the tiles, then the bias."""
    lead = x.shape[:-1]
    a = x.reshape(-1, x.shape[-1]).float()
    wf = w.float()
    m, k = a.shape
    n = wf.shape[0]
    aq, sa = quantise_activations_e4m3(a, q_max, tile_k)
    wq, sw = quantise_weights_e4m3(wf, q_max, tile_k, block_n)
    out = torch.zeros((m, n), dtype=torch.float32)
    accs = []
    for t, lo in enumerate(range(0, k, tile_k)):
        if TILE_SUM_EXACT:
            part = (aq[:, lo:lo + tile_k].double() @ wq[:, lo:lo + tile_k].double().T).float()
        else:
            part = aq[:, lo:lo + tile_k] @ wq[:, lo:lo + tile_k].T
        if taps is not None:
            accs.append(part.clone())
        part = part * sa[:, t:t + 1]
        part = part * sw[:, t].repeat_interleave(block_n)[None, :]
        out += part
    if taps is not None:
        taps.setdefault("qa_" + name, []).append(aq.clone())
        taps.setdefault("sa_" + name, []).append(sa.clone())
        taps.setdefault("acc_" + name, []).append(torch.stack(accs))
        # the quotients x / s before rounding to e4m3, in float64: how far each byte was from a tie
        taps.setdefault("quot_" + name, []).append(a.to(torch.float64) / sa.to(torch.float64).repeat_interleave(tile_k, dim=1))
    if bias is not None:
        out = out + bias.float()
    return out.reshape(*lead, n).to(x.dtype)


def _linear(x, w, b, mode, unsigned=False, taps=None, name=""):
    if mode == "int8":
        return int8_linear(x, w, b, unsigned, taps, name)
    if mode == "e4m3":
        return fp8_linear(x, w, b, taps, name)
    return F.linear(x, w, b)


def n_layers_of(sd) -> int:
    n = 0
    while f"encoder.layers.{n}.linear1.weight" in sd:
        n += 1
    return n


def value_from(sd: Dict[str, torch.Tensor], h, h_raw, control, alive, eps: float = 1e-5):
    """The value in [-1, 1] from the side to move's point of view (brokefish/nn/model.py:551-617).
    ``h`` is the stream after ``norm_f``, ``h_raw`` before it.  The head is the one the state_dict's
    ``value_mode`` marker names (absent: the king row): king = the mover's king token; pooled
    (1) = mean of the live tokens of ``h``; prenorm (2) = ``norm_f`` of the mean of the live tokens
    of ``h_raw``.  The pooled heads predict in White's frame and are negated for Black to move."""
    n, d = h.shape[0], h.shape[-1]
    vmode = int(sd["value_mode"]) if "value_mode" in sd else 0
    if vmode == 2:
        m = alive.unsqueeze(-1).to(h_raw.dtype)
        hv = F.layer_norm((h_raw * m).sum(1) / m.sum(1).clamp(min=1), (d,), sd["norm_f.weight"], sd["norm_f.bias"], eps)
    elif vmode == 1:
        m = alive.unsqueeze(-1).to(h.dtype)
        hv = (h * m).sum(1) / m.sum(1).clamp(min=1)
    else:
        king = torch.where(control < 0, KING_BLACK, KING_WHITE).to(torch.int64)
        hv = h[torch.arange(n), king]
    raw = F.linear(hv, sd["value.weight"]).float()
    if raw.shape[-1] == 1:
        value = torch.tanh(raw).squeeze(-1)
    else:  # classes 0 = loss, 1 = draw, 2 = win (brokefish/nn/model.py:156-170)
        pr = torch.softmax(raw, dim=-1)
        value = pr[:, 2] - pr[:, 0]
    if vmode:
        value = torch.where(control > 0, value, -value)
    return value


def forward(sd: Dict[str, torch.Tensor], boards, control, rep, mode: str = "int8",
            mask: Optional[torch.Tensor] = None, n_heads: Optional[int] = None,
            eps: float = 1e-5, taps: Optional[dict] = None,
            x_in: Optional[torch.Tensor] = None, layer_begin: int = 0,
            layer_end: Optional[int] = None):
    """(policy [N,32,64], promo [N,32,4], value [N]) in fp32, plus ``best`` [N] int64
    (slot*64+square of the masked argmax) when ``mask`` is given.

    ``mode`` is ``"fp32"`` (every matmul an ordinary ``F.linear``), ``"int8"`` (the four
    body matmuls of every layer through :func:`int8_linear`) or ``"e4m3"`` (through
    :func:`fp8_linear`).  ``x_in`` replaces the embedding as the residual stream entering
    layer ``layer_begin``; layers ``[layer_begin, layer_end)`` run (teacher forcing).
    """
    if mode not in ("fp32", "int8", "e4m3"):
        raise ValueError(mode)
    x, alive = embed(sd, boards, control, rep)
    if x_in is not None:
        x = x_in.clone()
    n, t, d = x.shape
    heads = n_heads if n_heads is not None else d // 32
    dh = d // heads
    if taps is not None:
        taps["embed"] = x.clone()
    key_bias = torch.zeros(n, 1, 1, t)
    key_bias.masked_fill_(~alive[:, None, None, :], float("-inf"))
    for i in range(layer_begin, n_layers_of(sd) if layer_end is None else layer_end):
        p = f"encoder.layers.{i}."
        y = F.layer_norm(x, (d,), sd[p + "norm1.weight"], sd[p + "norm1.bias"], eps)
        qkv = _linear(y, sd[p + "self_attn.in_proj_weight"], sd[p + "self_attn.in_proj_bias"],
                      mode, False, taps, "qkv")
        q, k, v = (z.reshape(n, t, heads, dh).transpose(1, 2) for z in qkv.split(d, dim=-1))
        s = (q @ k.transpose(-1, -2)) * (1.0 / math.sqrt(dh)) + key_bias
        o = (torch.softmax(s, dim=-1) @ v).transpose(1, 2).reshape(n, t, d)
        x = x + _linear(o, sd[p + "self_attn.out_proj.weight"], sd[p + "self_attn.out_proj.bias"],
                        mode, False, taps, "out")
        y = F.layer_norm(x, (d,), sd[p + "norm2.weight"], sd[p + "norm2.bias"], eps)
        hid = torch.relu(_linear(y, sd[p + "linear1.weight"], sd[p + "linear1.bias"],
                                 mode, False, taps, "ff1"))
        x = x + _linear(hid, sd[p + "linear2.weight"], sd[p + "linear2.bias"],
                        mode, True, taps, "ff2")
        if taps is not None:
            taps.setdefault("resid", []).append(x.clone())
    h = F.layer_norm(x, (d,), sd["norm_f.weight"], sd["norm_f.bias"], eps)
    if taps is not None:
        taps["normed"] = h.clone()
    policy = F.linear(h, sd["policy.weight"])
    promo = F.linear(h, sd["promo.weight"])
    value = value_from(sd, h, x, control, alive, eps)
    if mask is None:
        return policy, promo, value
    legal = ((mask.to(torch.int64)[..., None] >> torch.arange(64)) & 1).bool()
    policy = policy.masked_fill(~legal, float("-inf"))
    best = policy.reshape(n, -1).argmax(dim=1)   # torch.argmax returns the first maximum
    return policy, promo, value, best


def forward_library_stack(sd: Dict[str, torch.Tensor], boards, control, rep, mode: str = "int8",
                          n_heads: Optional[int] = None, eps: float = 1e-5, taps: Optional[dict] = None):
    """The same forward, but with the encoder stack run by torch's own
    ``nn.TransformerEncoder`` / ``nn.MultiheadAttention`` modules, exactly the modules the
    reference model is built from (brokefish/nn/model.py:303-311).

    In ``"int8"`` (``"e4m3"``) mode the four body matmuls of every layer are diverted to
    :func:`int8_linear` (:func:`fp8_linear`) by intercepting ``torch.nn.functional.linear`` for precisely those
    weight tensors (the only hook torch's attention module offers for its packed QKV and
    output projections), with the attention fast path switched off so the module really
    calls ``F.linear``; ``linear2`` gets the unsigned quantiser.  Under the torch version
    that wrote ``tests/golden/reference_vectors.npz`` this reproduces the reference's
    emulated forward bit for bit, which is what pins the composition.  ``taps`` (int8 mode)
    collects, per layer, the operand bytes, accumulators and float64 quotients of the four
    diverted matmuls under the names ``forward`` uses (``qa_qkv`` ... ``quot_ff2``).
    """
    from torch import nn

    x, alive = embed(sd, boards, control, rep)
    d = x.shape[-1]
    heads = n_heads if n_heads is not None else d // 32
    n_layers = n_layers_of(sd)
    f = sd["encoder.layers.0.linear1.weight"].shape[0]
    layer = nn.TransformerEncoderLayer(d_model=d, nhead=heads, dim_feedforward=f, batch_first=True,
                                       norm_first=True, dropout=0.0, layer_norm_eps=eps)
    stack = nn.TransformerEncoder(layer, num_layers=n_layers, norm=None, enable_nested_tensor=False).eval()
    stack.load_state_dict({k[len("encoder."):]: v for k, v in sd.items() if k.startswith("encoder.")})
    unsigned_of, name_of = {}, {}
    for lay in stack.layers:
        unsigned_of[id(lay.self_attn.in_proj_weight)] = False
        unsigned_of[id(lay.self_attn.out_proj.weight)] = False
        unsigned_of[id(lay.linear1.weight)] = False
        unsigned_of[id(lay.linear2.weight)] = True
        name_of.update({id(lay.self_attn.in_proj_weight): "qkv", id(lay.self_attn.out_proj.weight): "out",
                        id(lay.linear1.weight): "ff1", id(lay.linear2.weight): "ff2"})
    plain_linear = F.linear
    hits = [0]

    def routed(inp, weight, bias=None):
        u = unsigned_of.get(id(weight))
        if u is None or mode == "fp32":
            return plain_linear(inp, weight, bias)
        hits[0] += 1
        if mode == "e4m3":
            return fp8_linear(inp, weight, bias)
        return int8_linear(inp, weight, bias, unsigned=u, taps=taps, name=name_of[id(weight)])

    fast = torch.backends.mha.get_fastpath_enabled()
    if mode != "fp32":
        torch.backends.mha.set_fastpath_enabled(False)
    F.linear = routed
    try:
        with torch.no_grad():
            h = stack(x, src_key_padding_mask=~alive)
    finally:
        F.linear = plain_linear
        torch.backends.mha.set_fastpath_enabled(fast)
    if mode != "fp32" and hits[0] != 4 * n_layers:
        raise AssertionError(f"{hits[0]} matmuls were diverted, expected {4 * n_layers}")
    if taps:
        # torch's attention module runs its two projections on [token, board, channel]; bring
        # their rows into the [board, token] order of everything else
        n, t = x.shape[0], x.shape[1]
        for name in ("qkv", "out"):
            for key in ("qa_", "quot_"):
                taps[key + name] = [v.view(t, n, -1).transpose(0, 1).reshape(n * t, -1) for v in taps[key + name]]
            taps["acc_" + name] = [v.view(v.shape[0], t, n, -1).transpose(1, 2).reshape(v.shape[0], n * t, -1) for v in taps["acc_" + name]]
    h_raw = h
    h = F.layer_norm(h_raw, (d,), sd["norm_f.weight"], sd["norm_f.bias"], eps)
    policy = plain_linear(h, sd["policy.weight"])
    promo = plain_linear(h, sd["promo.weight"])
    return policy, promo, value_from(sd, h, h_raw, control, alive, eps)
