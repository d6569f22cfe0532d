"""``brokefish_amd.sync``: the weight-snapshot bookkeeping of the reference's training loop
(brokefish/train/sync.py:34-106) for the HIP evaluator.

``weight_fingerprint`` is pinned by the value the reference's own function returned for the
formula-weight network (tests/golden/make_golden.py) and by its defining properties: it moves
when a value moves and when two values swap places.
"""
import numpy as np
import pytest
import torch

import make_golden as mg
from brokefish_amd import sync
from brokefish_amd.net import BrokefishNet


def _golden_net():
    torch.manual_seed(0)
    net = BrokefishNet(n_value=1).eval()
    net.load_state_dict(mg.fill_state_dict(net.state_dict()))
    return net


def test_fingerprint_equals_the_references(golden):
    assert sync.weight_fingerprint(_golden_net()) == float(golden["weight_fingerprint_nv1"])


def test_fingerprint_sees_a_changed_value_and_a_permutation():
    net = _golden_net()
    f0 = sync.weight_fingerprint(net)
    with torch.no_grad():
        w = net.encoder.layers[3].linear1.weight
        a, b = w[5, 7].item(), w[5, 8].item()
        assert a != b
        w[5, 7], w[5, 8] = b, a                      # same multiset of values, other order
    f1 = sync.weight_fingerprint(net)
    with torch.no_grad():
        w[5, 7], w[5, 8] = a, b
        net.norm_f.bias[0] += 1e-3
    f2 = sync.weight_fingerprint(net)
    assert f1 != f0 and f2 != f0 and f2 != f1


def test_pack_argument_rules_do_not_need_a_gpu():
    net = BrokefishNet(n_layers=1)
    with pytest.raises(ValueError):
        sync.PackedWeights.pack(net, 0, fp8=True, int8=True)
    with pytest.raises(ValueError):
        sync.PackedWeights.pack(net, 0, impl="cuda", int8=True)


@pytest.mark.gpu
def test_a_stale_snapshot_is_refused():
    from brokefish_amd import positions
    net = _golden_net()
    packed = sync.PackedWeights.pack(net, weight_gen=3, int8=True)
    packed.assert_current(net, 3)
    b, c, r, _ = positions.random_positions(8, plies=40, seed=1)
    policy, promo, value = packed.evaluate()(b.cuda(), c.cuda(), r.cuda())
    assert policy.dtype is torch.float16 and policy.shape == (8, 32, 64) and value.dtype is torch.float32
    before = policy.clone()
    with pytest.raises(AssertionError, match="generation 3"):
        packed.assert_current(net, 4)
    with torch.no_grad():
        net.policy.weight[0, 0] += 0.5                # a gradient step outside the loop's accounting
    with pytest.raises(AssertionError, match="fingerprint"):
        packed.assert_current(net, 3)
    # the snapshot still evaluates the OLD weights: that is exactly why the check exists
    assert torch.equal(packed.evaluate()(b.cuda(), c.cuda(), r.cuda())[0], before)
    fresh = sync.PackedWeights.pack(net, weight_gen=4, fp8=True)
    fresh.assert_current(net, 4)
    assert fresh.encoder.fp8 and not torch.equal(fresh.evaluate()(b.cuda(), c.cuda(), r.cuda())[0], before)


def test_checkpoint_conventions_size_a_net_from_a_bare_state_dict():
    # reference brokefish/nn/model.py:173-248: the value width from value.weight, the variants from
    # optional marker buffers whose absence is the legacy answer
    from brokefish_amd import net as bn
    for d, heads, layers, nv in ((256, 8, 8, 1), (256, 8, 3, 3), (512, 16, 2, 1)):
        src = BrokefishNet(d_model=d, n_heads=heads, d_ff=4 * d, n_layers=layers, n_value=nv)
        state = src.state_dict()
        assert bn.n_value_of(state) == nv and bn.value_head_of(state) == "king"
        assert bn.reinject_of(state) == "none" and bn.rule_features_of(state) is False
        dst = bn.net_for_state(state)
        dst.load_state_dict(state, strict=True)
        assert (dst.d_model, dst.n_layers, dst.n_value) == (d, layers, nv)
        assert sync.weight_fingerprint(dst) == sync.weight_fingerprint(src)
    state = BrokefishNet(n_layers=1).state_dict()
    with pytest.raises(KeyError):
        bn.n_value_of({k: v for k, v in state.items() if k != "value.weight"})
    for key, val, fn in (("value_mode", 1, "pooled"), ("value_mode", 2, "prenorm")):
        marked = dict(state, **{key: torch.tensor(val)})
        assert bn.value_head_of(marked) == fn
        dst = bn.net_for_state(marked)                     # the pooled heads are carried: the marker rides along
        dst.load_state_dict(marked, strict=True)
        assert dst.value_head == fn and int(dst.state_dict()["value_mode"]) == val
    for key, val in (("reinject_mode", 1), ("rule_features_mode", 1)):
        with pytest.raises(NotImplementedError):
            bn.net_for_state(dict(state, **{key: torch.tensor(val)}))    # recognised, and loudly not carried
    assert bn.reinject_of(dict(state, reinject_mode=torch.tensor(2))) == "both"
    assert bn.rule_features_of(dict(state, rule_features_mode=torch.tensor(1))) is True
    with pytest.raises(ValueError):
        bn.value_head_of(dict(state, value_mode=torch.tensor(9)))
    with pytest.raises(ValueError):
        bn.rule_features_of(dict(state, rule_features_mode=torch.tensor(2)))


def test_master_network_forward_is_the_fp32_restatement_and_the_references_golden(golden):
    # brokefish_amd.net.BrokefishNet.forward against the checker's fp32 route and against the logits
    # the reference's own model wrote for the formula weights (brokefish/nn/model.py:621-645)
    import make_golden as mg
    from oracle import emulated
    for head, nv in (("king", 1), ("king", 3), ("pooled", 3), ("prenorm", 1)):
        torch.manual_seed(0)
        net = BrokefishNet(n_value=nv, value_head=head).eval()
        net.load_state_dict(mg.fill_state_dict(net.state_dict()))
        b, c, r = mg.positions()
        with torch.no_grad():
            got = net(b, c, r)
            want = emulated.forward({k: v for k, v in net.state_dict().items()}, b, c, r, mode="fp32")
        for g, w in zip(got, want):
            assert (g - w).abs().max() < 2e-5
        if head == "king":
            nb = 3 if nv == 3 else 8
            assert np.abs(got[0].numpy()[:nb] - golden[f"fp32_policy_nv{nv}"]).max() < 2e-5
            assert np.abs(got[2].numpy()[:nb] - golden[f"fp32_value_nv{nv}"]).max() < 2e-6
    m = torch.full((8, 32), 0x0F0F, dtype=torch.int64)
    with torch.no_grad():
        raw, pm, plain = net(b, c, r, mask=m)[0], net.forward_masked(b, c, r, m)[0], net(b, c, r)[0]
    assert torch.isfinite(raw).all() and torch.equal(raw, plain)                 # forward ignores the mask, as the reference's
    assert torch.isneginf(pm[:, :, 4]).all() and torch.equal(pm[:, :, 0], raw[:, :, 0])


@pytest.mark.gpu
def test_start_up_consistency_check_catches_a_stale_snapshot_a_nan_and_a_wrong_slab():
    # reference brokefish/train/loop.py:1109-1166 (check 9 of its training loop)
    for kw in ({"int8": True}, {"fp8": True}):
        torch.manual_seed(0)
        net = BrokefishNet().eval()
        packed = sync.PackedWeights.pack(net, 0, **kw)
        fp_before = sync.weight_fingerprint(net)
        res = sync.check_weights_propagate(net, packed)
        assert res["moved"] > 0 and res["agree"] <= res["tol"] and sync.weight_fingerprint(net) == fp_before
    # a stale snapshot: packing hands back the evaluator of the old weights
    real_pack = sync.PackedWeights.pack
    try:
        sync.PackedWeights.pack = classmethod(lambda cls, *a, **k: packed)
        with pytest.raises(AssertionError, match="did not change"):
            sync.check_weights_propagate(net, packed)
        # a wrong weight slab: the repacked evaluator holds another network's weights
        torch.manual_seed(7)
        other = real_pack(BrokefishNet().eval().randomise_layers_(seed=8, scale=3.0), 1, int8=True)
        sync.PackedWeights.pack = classmethod(lambda cls, *a, **k: other)
        with pytest.raises(AssertionError, match="disagrees"):
            sync.check_weights_propagate(net, packed)
    finally:
        sync.PackedWeights.pack = real_pack
    # a non-finite output is an error, not a pass (nan > tol is False)
    torch.manual_seed(0)
    bad = BrokefishNet().eval()
    with torch.no_grad():
        bad.norm_f.weight[3] = float("nan")
    with pytest.raises(AssertionError, match="non-finite"):
        sync.check_weights_propagate(bad, sync.PackedWeights.pack(bad, 0, int8=True))
