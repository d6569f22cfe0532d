"""TEST INFRASTRUCTURE -- NOT PRODUCT CODE.

A CPU restatement, in float64 numpy, of the edge expansion the reference's search performs on
the evaluator's outputs (docs/reference/search.md:616-636, steps 2-6; the torch code it follows is
brokefish/search/torch_impl.py:962-1033 with `_promotion_targets` at :948-960).  Only ``tests/``
imports this module.

Pins (tests/test_expand.py): what the reference's own ``Search._expand`` wrote for 38 positions
(the eight golden positions and the reference's edge-case positions, 218 candidates among them) at
E = 96 and E = 16 with formula logits (tests/golden/reference_vectors_expand.npz, written by
``tests/golden/make_golden.py expand``): move codes, edge and candidate counts exactly, priors to
fp16 rounding, truncated mass to 2e-6; the canonical order and the four-way promotion fan-out on hand-built
positions, the properties the reference's own tests assert (tests/test_search.py:317-372: order
sorted by (move, type), edges = mask bits + 3 per promoting move, priors sum to 1, nothing beyond
n_edges, the four edges of a promoting move split its mass by softmax(promo), truncation keeps
exactly E edges and reports a positive dropped mass), and brute-force definitions on small cases
(the kept set is the E largest log-priors with ties by order; dropped = 1 - kept mass under the
untruncated softmax).
"""
from __future__ import annotations

import numpy as np

PAWN = 0            # docs/reference/spec.md:47
MOVE_BITS = 11      # brokefish/search/torch_impl.py:61
PROMO_SHIFT = 11    # brokefish/search/torch_impl.py:62


def candidates(board_words, control, mask_words):
    """[(move, type)] of one position in canonical order: ascending slot, then square; a live
    pawn's move onto the last rank of the side to move expands to types 0..3 (N B R Q)."""
    last_rank = 0 if control < 0 else 7
    out = []
    for p in range(32):
        w = int(board_words[p]) & 0xFFFF
        pawn = ((w >> 11) & 1) == 0 and ((w >> 6) & 7) == PAWN
        m = int(mask_words[p]) & 0xFFFFFFFFFFFFFFFF
        for s in range(64):
            if (m >> s) & 1:
                if pawn and s // 8 == last_rank:
                    out += [(p * 64 + s, k) for k in range(4)]
                else:
                    out.append((p * 64 + s, 0))
    return out


def expand(policy, promo, value, mask, boards, control, max_edges: int = 96):
    """numpy in, dict out: edge_move [n,E] int16, edge_prior [n,E] float64 (exact, unrounded),
    n_edges [n], count [n], dropped [n] float64, node_value [n] float64, and `margin` [n]: the gap
    between the last kept and the first dropped log-prior (inf without truncation)."""
    policy = np.asarray(policy, np.float64)
    promo = np.asarray(promo, np.float64)
    n, E = policy.shape[0], max_edges
    out = {"edge_move": np.zeros((n, E), np.int16), "edge_prior": np.zeros((n, E), np.float64),
           "n_edges": np.zeros(n, np.int32), "count": np.zeros(n, np.int32),
           "dropped": np.zeros(n, np.float64), "margin": np.full(n, np.inf),
           "node_value": (np.asarray(value, np.float64) + 1.0) / 2.0}
    x = promo - promo.max(-1, keepdims=True)
    lp = x - np.log(np.exp(x).sum(-1, keepdims=True))                  # log_softmax, [n,32,4]
    for b in range(n):
        cand = candidates(np.asarray(boards[b]).view(np.uint16) if np.asarray(boards[b]).dtype == np.int16
                          else boards[b], int(control[b]), np.asarray(mask[b]).view(np.uint64)
                          if np.asarray(mask[b]).dtype == np.int64 else mask[b])
        out["count"][b] = len(cand)
        if not cand:
            continue
        # a promotion edge is recognised by its move having four entries
        is_promo = {}
        for mv, k in cand:
            is_promo[mv] = is_promo.get(mv, 0) + 1
        logit = np.array([policy[b, mv // 64, mv % 64] + (lp[b, mv // 64, k] if is_promo[mv] == 4 else 0.0)
                          for mv, k in cand])
        keep = np.ones(len(cand), bool)
        if len(cand) > E:
            order = np.argsort(-logit, kind="stable")                  # ties by canonical order
            keep[:] = False
            keep[order[:E]] = True
            before = np.exp(logit - logit.max())
            before /= before.sum()
            out["dropped"][b] = before[~keep].sum()
            out["margin"][b] = logit[order[E - 1]] - logit[order[E]]
        kl = logit[keep]
        pr = np.exp(kl - kl.max())
        pr /= pr.sum()
        ne = int(keep.sum())
        out["n_edges"][b] = ne
        codes = [mv | (k << PROMO_SHIFT) for (mv, k), kp in zip(cand, keep) if kp]
        out["edge_move"][b, :ne] = np.array(codes, np.int64).astype(np.int16)
        out["edge_prior"][b, :ne] = pr
    return out
