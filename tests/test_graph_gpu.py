"""The device chain (move generation -> evaluator -> edge expansion) under HIP graph capture.

Small launches are latency-bound (a 64-position evaluation is 0.12 ms of kernel time), so a search
would capture the chain once and replay it.  None of the three entry points allocates, waits on
the host or clears memory with a memset node, so the chain can be captured as it is.  Each replay
is checked against the eager chain on the same inputs, with eager work and synchronisations
between the replays.
"""
import pytest
import torch

from brokefish_amd import encoder_impl, positions
from brokefish_amd.net import BrokefishNet

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [64, 700])
def test_captured_chain_replays_bit_identically_to_the_eager_chain(n):
    torch.manual_seed(0)
    net = BrokefishNet().eval()
    model = encoder_impl("hip")(net, int8=True)
    eager_model = encoder_impl("hip")(net, int8=True)
    b, c, r, _ = positions.random_positions(n, plies=120, seed=40)
    sb, sc, sr = b.cuda(), c.cuda(), r.cuda()                 # the graph's static inputs

    side = torch.cuda.Stream()                                 # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            model.forward_expand(sb, sc, sr)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        edges = model.forward_expand(sb, sc, sr)
    keys = ("edge_move", "edge_prior", "n_edges", "count", "dropped", "node_value", "mask", "in_check")

    for seed in (41, 42, 43):
        b, c, r, m = positions.random_positions(n, plies=120, seed=seed)
        sb.copy_(b), sc.copy_(c), sr.copy_(r)
        graph.replay()
        torch.cuda.synchronize()
        got = {k: edges[k].clone() for k in keys}
        logits = [t.clone() for t in (model.policy_out, model.promo_out, model.value_out)]
        want = eager_model.forward_expand(b.cuda(), c.cuda(), r.cuda())       # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(got["mask"].cpu(), m), seed
        for k in keys:
            assert torch.equal(got[k], want[k]), (seed, k)
        for g_, w_ in zip(logits, (eager_model.policy_out, eager_model.promo_out, eager_model.value_out)):
            assert torch.equal(g_, w_), seed
