"""Prior-space comparison of two sets of logits: how the reference itself holds a kernel to its
emulation (reference brokefish/nn/validate.py:249-388; the numbers it publishes are in
docs/ledger/perf.md:684-693: max |dp|, its 95th percentile, how often the top-1 move changes and
how often the largest prior error exceeds the gap between the two best moves).

A logit error matters through the prior the search builds from it, so both sets of logits are
pushed through the search's expand step on the device (:func:`brokefish_amd.hip_impl.expand_edges`:
legal-move mask, promotion log-softmax, truncation to ``max_edges``, softmax) and the priors are
compared edge by edge.  Positions whose surviving edge sets differ are counted separately and
left out of the differences, as the reference does.
"""
from __future__ import annotations

from dataclasses import dataclass, asdict

import torch

from . import hip_impl


@dataclass
class Delta:
    """One comparison (field meanings as reference brokefish/nn/validate.py:291-312)."""
    name: str
    positions: int
    max_abs: float          # largest |p_got - p_ref| over all legal edges
    p95_abs: float          # 95th percentile of the same
    top1_disagree: float    # share of positions whose most probable move changed
    flip_risk: float        # share whose largest prior error exceeds the reference's top-two gap
    edge_set_differs: int   # positions where truncation kept different edges (left out above)
    max_abs_value: float    # largest |value_got - value_ref|
    nonfinite: int

    def as_dict(self):
        return asdict(self)


def priors(policy, promo, value, mask, boards, control, max_edges: int = 96):
    """(prior [n,E] fp32, move [n,E] int16, n_edges [n]) from logits, through the device expand step."""
    out = hip_impl.expand_edges(policy, promo, value, mask, boards, control, max_edges=max_edges)
    return out["edge_prior"].float(), out["edge_move"], out["n_edges"].long()


@torch.no_grad()
def compare(name: str, ref, got, mask, boards, control, max_edges: int = 96) -> Delta:
    """``ref`` and ``got`` are ``(policy [n,32,64], promo [n,32,4], value [n])`` on the GPU (fp16 or
    fp32 logits); ``mask`` the legal-move words of the positions."""
    p_ref, m_ref, ne_ref = priors(ref[0], ref[1], ref[2].float(), mask, boards, control, max_edges)
    p_got, m_got, ne_got = priors(got[0], got[1], got[2].float(), mask, boards, control, max_edges)
    e = p_ref.shape[1]
    valid = torch.arange(e, device=p_ref.device)[None, :] < ne_ref[:, None]
    same_set = (ne_ref == ne_got) & ((m_ref == m_got) | ~valid).all(-1)
    v = valid & same_set[:, None]
    d = torch.where(v, (p_got - p_ref).abs(), torch.zeros_like(p_ref))
    flat = d[v]
    neg = torch.finfo(torch.float32).min
    a = torch.where(v, p_ref, torch.full_like(p_ref, neg))
    b = torch.where(v, p_got, torch.full_like(p_got, neg))
    rows = same_set & (ne_ref > 0)
    n = max(int(rows.sum()), 1)
    two = a.topk(min(2, e), dim=-1).values
    gap = two[:, 0] - two[:, 1] if two.shape[1] == 2 else torch.ones_like(two[:, 0])
    gap = torch.where(ne_ref > 1, gap, torch.ones_like(gap))
    nonfinite = sum(int((~torch.isfinite(t.float())).sum()) for t in (got[1], got[2])) + \
        int(torch.isnan(got[0].float()).sum())        # masked policy entries are -inf by contract
    return Delta(name=name, positions=int(p_ref.shape[0]),
                 max_abs=float(d.max()) if bool(v.any()) else float("inf"),
                 p95_abs=float(torch.quantile(flat[:2 ** 24], 0.95)) if flat.numel() else float("inf"),
                 top1_disagree=float((a.argmax(-1) != b.argmax(-1))[rows].sum()) / n,
                 flip_risk=float((d.max(-1).values > gap)[rows].sum()) / n,
                 edge_set_differs=int((~same_set).sum()),
                 max_abs_value=float((got[2].float() - ref[2].float()).abs().max()),
                 nonfinite=nonfinite)
