"""The network whose weights the evaluator runs: a weight container with the reference's
``state_dict`` key names, so reference checkpoints load unchanged.

Same constructor arguments, parameter names and initialisation rules as the reference
model (brokefish/nn/model.py:276-361): five embedding tables, a pre-norm ReLU
``nn.TransformerEncoder`` (deep-copied layers, so a fresh net holds identical layers), a
final LayerNorm, and three biasless heads; embeddings and heads N(0, 1/sqrt(d)).

The evaluator only *reads* parameters from it (``FusedEncoder(net)`` snapshots them).
Only the king value head and no re-injection / rule features are carried: those are the
defaults every published number of the reference uses.
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
        if value_head != "king" or reinject != "none" or rule_features:
            raise NotImplementedError(
                "only the king value head without re-injection or rule features is carried")
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
        std = d_model ** -0.5
        for mod in (self.emb_square, self.emb_type_special, self.emb_color_turn, self.emb_clock,
                    self.emb_rep, self.policy, self.promo, self.value):
            nn.init.normal_(mod.weight, mean=0.0, std=std)

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
