"""The network whose weights the evaluator runs: a weight container with the reference's
``state_dict`` key names, so reference checkpoints load unchanged.

Same constructor arguments, parameter names and initialisation rules as the reference
model (brokefish/nn/model.py:276-361): five embedding tables, a pre-norm ReLU
``nn.TransformerEncoder`` (deep-copied layers, so a fresh net holds identical layers), a
final LayerNorm, and three biasless heads; embeddings and heads N(0, 1/sqrt(d)).

The evaluator only *reads* parameters from it (``FusedEncoder(net)`` snapshots them);
``forward`` is the plain PyTorch master network a trainer differentiates.
The three value heads (king row, pooled, prenorm) are carried; re-injection and rule
features are not (the defaults every published number of the reference uses).
"""
from __future__ import annotations

import torch
from torch import nn

D_MODEL, N_LAYERS, N_HEADS, D_FF, T = 256, 8, 8, 1024, 32
N_SQUARE, N_TYPE_SPECIAL, N_COLOR_TURN, N_CLOCK, N_REP = 64, 12, 4, 101, 3
N_POLICY, N_PROMO = 64, 4
KING_SLOT_WHITE, KING_SLOT_BLACK = 15, 31


class BrokefishNet(nn.Module):
    def __init__(self, d_model: int = D_MODEL, n_layers: int = N_LAYERS, n_heads: int = N_HEADS,
                 d_ff: int = D_FF, eps: float = 1e-5, n_value: int = 1, value_head: str = "king",
                 reinject: str = "none", rule_features: bool = False):
        super().__init__()
        if n_value not in (1, 3):
            raise ValueError(f"n_value must be 1 (scalar tanh) or 3 (win/draw/loss), got {n_value}")
        if value_head not in VALUE_HEADS:
            raise ValueError(f"value_head must be one of {VALUE_HEADS}, got {value_head!r}")
        if reinject != "none" or rule_features:
            raise NotImplementedError("re-injection and rule features are not carried")
        self.d_model, self.n_layers, self.n_value = d_model, n_layers, n_value
        self.value_head, self.reinject, self.rule_features = value_head, reinject, False
        self.emb_square = nn.Embedding(N_SQUARE, d_model)
        self.emb_type_special = nn.Embedding(N_TYPE_SPECIAL, d_model)
        self.emb_color_turn = nn.Embedding(N_COLOR_TURN, d_model)
        self.emb_clock = nn.Embedding(N_CLOCK, d_model)
        self.emb_rep = nn.Embedding(N_REP, d_model)
        layer = nn.TransformerEncoderLayer(d_model=d_model, nhead=n_heads, dim_feedforward=d_ff,
                                           batch_first=True, norm_first=True, dropout=0.0,
                                           layer_norm_eps=eps)
        self.encoder = nn.TransformerEncoder(layer, num_layers=n_layers, norm=None,
                                             enable_nested_tensor=False)
        self.norm_f = nn.LayerNorm(d_model, eps=eps)
        self.policy = nn.Linear(d_model, N_POLICY, bias=False)
        self.promo = nn.Linear(d_model, N_PROMO, bias=False)
        self.value = nn.Linear(d_model, n_value, bias=False)
        # the marker rides in the state_dict only for the pooled heads: its absence is the king
        # head of every older checkpoint (brokefish/nn/model.py:318-331)
        if value_head in VALUE_MODE_ID:
            self.register_buffer("value_mode", torch.tensor(VALUE_MODE_ID[value_head], dtype=torch.int64))
        std = d_model ** -0.5
        for mod in (self.emb_square, self.emb_type_special, self.emb_color_turn, self.emb_clock,
                    self.emb_rep, self.policy, self.promo, self.value):
            nn.init.normal_(mod.weight, mean=0.0, std=std)

    def forward(self, boards, control, rep, mask=None):
        """The master network in plain PyTorch, in the parameters' dtype and on their device
        (reference brokefish/nn/model.py:621-645): ``boards [n,32]`` int16 words, ``control [n]``
        int16, ``rep [n]`` uint8 -> ``(policy [n,32,64], promo [n,32,4], value [n])``, raw logits.
        ``mask`` is accepted and ignored, as in the reference (rule features are not carried here,
        and without them its ``forward`` never reads the mask: "a caller may always pass what it
        has"); :meth:`forward_masked` is the variant that sets illegal entries to -inf.  This is
        what a trainer differentiates and what :func:`brokefish_amd.sync.check_weights_propagate`
        holds a packed evaluator against; the evaluator itself never calls it."""
        w = boards.to(torch.int64) & 0xFFFF
        alive = ((w >> 11) & 1) == 0
        stm = (control < 0).to(torch.int64)
        i_ts = (((w >> 6) & 7) * 2 + ((w >> 9) & 1)).clamp(max=N_TYPE_SPECIAL - 1)
        i_ct = ((w >> 10) & 1) * 2 + stm[:, None]
        i_clock = (control.to(torch.int64).abs() - 1).clamp(0, N_CLOCK - 1)
        i_rep = rep.to(torch.int64).clamp(0, N_REP - 1)
        per_board = self.emb_clock(i_clock) + self.emb_rep(i_rep)          # the order of spec 7.2
        x = self.emb_square(w & 63)
        x = x + self.emb_type_special(i_ts)
        x = x + self.emb_color_turn(i_ct)
        x = x + per_board[:, None, :]
        h_raw = self.encoder(x, src_key_padding_mask=~alive)
        h = self.norm_f(h_raw)
        if self.value_head == "prenorm":
            m = alive.unsqueeze(-1).to(h_raw.dtype)
            hv = self.norm_f((h_raw * m).sum(1) / m.sum(1).clamp(min=1))
        elif self.value_head == "pooled":
            m = alive.unsqueeze(-1).to(h.dtype)
            hv = (h * m).sum(1) / m.sum(1).clamp(min=1)
        else:
            king = torch.where(control < 0, KING_SLOT_BLACK, KING_SLOT_WHITE).to(torch.int64)
            hv = h[torch.arange(h.shape[0], device=h.device), king]
        raw = self.value(hv).float()
        if self.n_value == 1:
            value = torch.tanh(raw).squeeze(-1)
        else:                                   # classes loss, draw, win: p(win) - p(loss)
            pr = torch.softmax(raw, dim=-1)
            value = pr[:, 2] - pr[:, 0]
        if self.value_head != "king":           # the pooled heads predict in White's frame
            value = torch.where(control > 0, value, -value)
        return self.policy(h), self.promo(h), value

    def forward_masked(self, boards, control, rep, mask):
        """``forward`` with the illegal policy entries set to -inf (``mask [n,32]`` int64 legal-move
        words, bit s of word p set iff p -> s is legal): what the evaluator's ``forward_masked``
        returns, for comparisons; not for a loss (0 * -inf is NaN)."""
        policy, promo, value = self.forward(boards, control, rep)
        legal = ((mask.to(torch.int64)[..., None] >> torch.arange(64, device=mask.device)) & 1).bool()
        return policy.masked_fill(~legal, float("-inf")), promo, value

    @torch.no_grad()
    def randomise_layers_(self, seed: int = 1, scale: float = 1.0) -> "BrokefishNet":
        """Give every layer its own weights, biases and LayerNorm affine.

        A freshly built net holds L copies of one layer with zero attention biases and
        identity norms, which hides layer-index, bias and affine mistakes from any test.
        """
        g = torch.Generator().manual_seed(seed)
        for lay in self.encoder.layers:
            for p in lay.parameters():
                if p.dim() == 2:
                    p.copy_(torch.randn(p.shape, generator=g) * (scale / p.shape[1] ** 0.5))
                elif "norm" in [n for n, q in lay.named_parameters() if q is p][0] and \
                        [n for n, q in lay.named_parameters() if q is p][0].endswith("weight"):
                    p.copy_(1.0 + 0.2 * torch.randn(p.shape, generator=g))
                else:
                    p.copy_(0.1 * torch.randn(p.shape, generator=g))
        self.norm_f.weight.copy_(1.0 + 0.2 * torch.randn(self.d_model, generator=g))
        self.norm_f.bias.copy_(0.1 * torch.randn(self.d_model, generator=g))
        return self


# --------------------------------------------------------------------------- #
# checkpoint conventions (reference brokefish/nn/model.py:173-248)
# --------------------------------------------------------------------------- #
# Checkpoints are bare state_dicts; what a file was trained with is recovered from the shape of
# `value.weight` and from optional marker buffers whose absence is the legacy answer.

VALUE_HEADS = ("king", "pooled", "prenorm")      # brokefish/nn/model.py:89
VALUE_MODE_ID = {"pooled": 1, "prenorm": 2}      # brokefish/nn/model.py:93
REINJECT_MODE_ID = {"ln1": 1, "both": 2}         # brokefish/nn/model.py:115
RULE_FEATURES_ID = 1                             # brokefish/nn/model.py:153


def n_value_of(state: dict) -> int:
    """How many value rows a ``state_dict`` was trained with (1: tanh scalar, 3: win/draw/loss)."""
    w = state.get("value.weight")
    if w is None:
        raise KeyError("no `value.weight` in this state_dict, so its value head cannot be sized. "
                       "Pass the network's weights, not a training checkpoint")
    return int(w.shape[0])


def _mode_of(state: dict, key: str, ids: dict, legacy: str) -> str:
    if key not in state:
        return legacy
    got = int(state[key])
    for name, i in ids.items():
        if i == got:
            return name
    raise ValueError(f"unknown {key} {got} in this state_dict; this build knows {ids}")


def value_head_of(state: dict) -> str:
    """Which value head a ``state_dict`` was written with; no marker means the king select."""
    return _mode_of(state, "value_mode", VALUE_MODE_ID, "king")


def reinject_of(state: dict) -> str:
    """Which per-layer input re-injection a ``state_dict`` was written with; no marker: none."""
    return _mode_of(state, "reinject_mode", REINJECT_MODE_ID, "none")


def rule_features_of(state: dict) -> bool:
    """Whether a ``state_dict`` carries the rule-derived piece inputs; no marker: it does not."""
    if "rule_features_mode" not in state:
        return False
    got = int(state["rule_features_mode"])
    if got != RULE_FEATURES_ID:
        raise ValueError(f"unknown rule_features_mode {got} in this state_dict; this build knows {RULE_FEATURES_ID}")
    return True


def net_for_state(state: dict, **kw) -> BrokefishNet:
    """An empty net shaped to hold ``state`` (load into it).  Width, depth and feed-forward width
    are read off the tensors unless given; a head or input variant this library does not carry
    raises ``NotImplementedError`` from the constructor."""
    n_layers = 0
    while f"encoder.layers.{n_layers}.linear1.weight" in state:
        n_layers += 1
    if not n_layers or "emb_square.weight" not in state:
        raise KeyError("not a network state_dict: no encoder layers / embedding tables in it")
    d_model = int(state["emb_square.weight"].shape[1])
    kw.setdefault("d_model", d_model)
    kw.setdefault("n_layers", n_layers)
    kw.setdefault("n_heads", d_model // 32)
    kw.setdefault("d_ff", int(state["encoder.layers.0.linear1.weight"].shape[0]))
    return BrokefishNet(n_value=n_value_of(state), value_head=value_head_of(state),
                        reinject=reinject_of(state), rule_features=rule_features_of(state), **kw)
