"""Pins the e4m3 part of ``oracle/emulated.py`` (the checker of the evaluator's fp8 variant).

=====================  ==========================================================================
function               pinned by
=====================  ==========================================================================
activation quantiser   the reference's own properties (tests/test_quant.py:43-68: the tile maximum
                       lands on q_max, nothing becomes NaN, 3 mantissa bits of relative error, a
                       zero tile stays zero with a positive scale); golden bytes + scales written
                       by the reference's quantise_activations
weight quantiser       two-dimensional blocks (tests/test_quant.py:71-84), refusal of shapes that
                       do not tile (:87-90); golden checksums + scales of quantise_weights_bytes
fp8_linear             exact closed form: operands already on the e4m3 grid with power-of-two
                       scales make every product and sum exact, so the result must equal the
                       float64 matrix product (the device KAT of csrc/tests/tfp8.cu does the same
                       against a host product); golden outputs of the reference's fp8_linear at
                       the shipped constants and at the module's 128-deep / 448 defaults
forward composition    golden logits/value of the reference's emulated_forward under the shipped
                       e4m3 constants, reproduced BIT FOR BIT by the library-stack route
=====================  ==========================================================================

Inside one k-tile the fp32 sum of 256 e4m3 products is not exact in general (the products
are multiples of 2^-18 and the sum can pass 2^6), so two implementations that order that
sum differently agree to rounding, not bit for bit; the GPU tests state their tolerance.
"""
import numpy as np
import pytest
import torch

import make_golden as mg
from brokefish_amd import hip_impl
from brokefish_amd.net import BrokefishNet
from oracle import emulated


@pytest.fixture(scope="module")
def golden8():
    import os
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors_e4m3.npz"))


@pytest.mark.parametrize("q_max", [448.0, 16.0, 8.0])
@pytest.mark.parametrize("tile_k", [32, 128, 256])
def test_activation_tiles_use_the_whole_range_and_never_nan(q_max, tile_k):
    torch.manual_seed(0)
    x = torch.randn(64, 256) * torch.logspace(-3, 2, 256)
    q, scale = emulated.quantise_activations_e4m3(x, q_max, tile_k)
    assert scale.shape == (64, 256 // tile_k)
    assert torch.isfinite(q).all()
    tiles = q.view(64, 256 // tile_k, tile_k).abs().amax(-1)
    live = tiles > 0
    assert float((tiles[live] - q_max).abs().max()) <= q_max * 0.13
    rel = (q * scale.repeat_interleave(tile_k, 1) - x).abs() / x.abs().clamp(min=1e-30)
    # 3 mantissa bits wherever the quotient is a normal e4m3 number (>= 2^-6); below that the
    # format goes subnormal, which is the stated price of a small q_max
    big = (x.abs() > x.abs().amax() * 1e-3) & ((x / scale.repeat_interleave(tile_k, 1)).abs() >= 2.0 ** -6)
    assert float(rel[big].max()) < 0.07


def test_an_all_zero_tile_stays_zero():
    q, scale = emulated.quantise_activations_e4m3(torch.zeros(4, 256), 8.0, 256)
    assert float(q.abs().max()) == 0.0 and float(scale.min()) == 1.0


def test_weight_blocks_are_two_dimensional():
    torch.manual_seed(0)
    w = torch.randn(256, 512)
    w[0, :] *= 100.0                       # one loud row inside block row 0
    q, scale = emulated.quantise_weights_e4m3(w, 448.0, 128, 128)
    assert scale.shape == (2, 4)
    back = q * scale.repeat_interleave(128, 0).repeat_interleave(128, 1)
    assert torch.isfinite(back).all()
    assert float(scale[0, 0]) > 10 * float(scale[1, 0])
    for bad in ((200, 256), (256, 200)):
        with pytest.raises(ValueError):
            emulated.quantise_weights_e4m3(torch.zeros(*bad), 448.0, 128, 128)
        with pytest.raises(ValueError):
            hip_impl.quantise_weights_e4m3(torch.zeros(*bad))


def test_fp8_linear_is_the_exact_product_on_grid_operands():
    # Operands on the e4m3 grid, every row / block holding +-8 so all scales are exactly 1:
    # products are multiples of 2^-6 below 64, sums of 256 of them stay below 2^14 and on a
    # 2^-6 grid, i.e. exact in fp32 in any order.  A dropped tile, a transposed operand or a
    # scale applied on the wrong axis all change the result.
    rng = np.random.default_rng(3)
    grid = np.array([0, 0.125, 0.25, 0.5, 0.75, 1, 1.25, 1.5, 1.75, 2, 2.5, 3, 3.5, 4, 5, 6, 7, 8], np.float32)
    a = rng.choice(grid, (32, 1024)) * rng.choice([-1.0, 1.0], (32, 1024))
    w = rng.choice(grid, (256, 1024)) * rng.choice([-1.0, 1.0], (256, 1024))
    for t in range(4):
        a[:, 256 * t] = 8.0
        w[0, 256 * t] = w[128, 256 * t] = -8.0
    bias = rng.integers(-4, 5, 256).astype(np.float32)
    taps = {}
    got = emulated.fp8_linear(torch.from_numpy(a.astype(np.float32)), torch.from_numpy(w.astype(np.float32)),
                              torch.from_numpy(bias), taps, "t")
    want = a.astype(np.float64) @ w.astype(np.float64).T + bias
    assert (got.numpy().astype(np.float64) == want).all()
    assert (taps["qa_t"][0].numpy() == a).all() and (taps["sa_t"][0].numpy() == 1.0).all()
    # distinct power-of-two scales per k-tile and per block on integer operands (products are
    # integers below 2^14 per tile, descale factors between 2^-3 and 2^4: every partial sum
    # fits 24 bits, so the result is still exact) -- a scale taken from the wrong tile or
    # block now shows
    a2 = np.rint(a)
    w2 = np.rint(w)
    for t in range(4):
        a2[:, 256 * t] = 8.0
        w2[0, 256 * t] = w2[128, 256 * t] = -8.0
        a2[:, 256 * t:256 * (t + 1)] *= 2.0 ** t
        w2[:128, 256 * t:256 * (t + 1)] *= 2.0 ** (t - 3)
        w2[128:, 256 * t:256 * (t + 1)] *= 2.0 ** (t % 2)
    got2 = emulated.fp8_linear(torch.from_numpy(a2.astype(np.float32)), torch.from_numpy(w2.astype(np.float32)), None)
    want2 = a2.astype(np.float64) @ w2.astype(np.float64).T
    assert (got2.numpy().astype(np.float64) == want2).all()


def test_golden_fp8_linear_and_quantisers(golden8):
    same_torch = str(golden8["torch_version"]) == torch.__version__
    for name, x, w, bias, _ in mg.linear_cases():
        got = emulated.fp8_linear(x, w, bias).numpy()
        got128 = emulated.fp8_linear(x, w, bias, q_max=448.0, tile_k=128).numpy()
        for g, key in ((got, "lin_"), (got128, "lin128_")):
            want = golden8[key + name]
            if same_torch:
                assert (g.view(np.int32) == want.view(np.int32)).all(), key + name
            else:   # another torch build may order the sum inside a tile differently
                assert np.abs(g - want).max() <= 1e-5 * np.abs(want).max(), key + name
        q, s = emulated.quantise_activations_e4m3(x[:, :256].contiguous())
        assert (q.to(torch.float8_e4m3fn).view(torch.uint8).numpy() == golden8["qa_" + name]).all()
        assert (s.numpy() == golden8["sa_" + name]).all()
        wb, ws = hip_impl.quantise_weights_e4m3(w)                     # what the host packs
        wq, ws2 = emulated.quantise_weights_e4m3(w)                    # what the checker multiplies
        assert (mg.weight_checksum(wb) == golden8["wqsum_" + name]).all()
        assert (ws == golden8["ws_" + name]).all() and (ws2.numpy() == ws).all()
        assert (wq.to(torch.float8_e4m3fn).view(torch.uint8).numpy() == wb).all()
    assert golden8["sa_s8_zero_row"][3, 0] == 1.0


def _golden_net():
    torch.manual_seed(0)
    net = BrokefishNet(n_value=1).eval()
    return (mg.fill_state_dict(net.state_dict()),) + tuple(mg.positions())


def test_golden_forward_e4m3_bit_exact_through_the_library_stack(golden, golden8):
    sd, b, c, r = _golden_net()
    got = emulated.forward_library_stack(sd, b, c, r, mode="e4m3")
    same_torch = str(golden8["torch_version"]) == torch.__version__
    for i, name in enumerate(("policy", "promo", "value")):
        want = golden8[f"e4m3_{name}_nv1"]
        if same_torch:
            assert (got[i].numpy().view(np.int32) == want.view(np.int32)).all(), name
        else:
            assert np.abs(got[i].numpy() - want).max() < 1e-1, name
    # the format's own error against fp32: the scale a tolerance has to be read against
    noise = np.abs(golden8["e4m3_policy_nv1"] - golden["fp32_policy_nv1"]).max()
    assert 1e-3 < noise < 1.0


def test_golden_forward_e4m3_functional_route(golden, golden8):
    # Same algorithm with attention written out (other fp32 summation order): agreement to
    # the forward's own sensitivity, far below the format's error against fp32.
    sd, b, c, r = _golden_net()
    with torch.no_grad():
        got = emulated.forward(sd, b, c, r, mode="e4m3")
    noise = np.abs(golden8["e4m3_policy_nv1"] - golden["fp32_policy_nv1"]).max()
    assert np.abs(got[0].numpy() - golden8["e4m3_policy_nv1"]).max() < noise
    assert np.abs(got[2].numpy() - golden8["e4m3_value_nv1"]).max() < 2e-2


def test_free_running_sensitivity_of_e4m3_is_a_property_of_the_algorithm():
    # The same torch code with the k-tile products summed exactly (float64, rounded once)
    # instead of in the library's fp32 order: operands differ only where a quotient sits within
    # fp32 rounding of an e4m3 tie, yet one such flip is 6 % of the element and moves a board's
    # logits by ~0.1.  So "logits within 2e-2" holds board by board only for boards without a
    # flip, for ANY two realisations of the formula that do not share a summation order; this is
    # the spread a kernel's free-running comparison has to be read against.
    from brokefish_amd import positions
    torch.manual_seed(0)
    net = BrokefishNet().eval()
    net.randomise_layers_(seed=3)
    sd = {k: v.detach() for k, v in net.state_dict().items()}
    b, c, r, _ = positions.random_positions(64, plies=120, seed=11, stamp_queen=True)
    with torch.no_grad():
        lib = emulated.forward(sd, b, c, r, mode="e4m3")
        with emulated.exact_tile_sums():
            exact = emulated.forward(sd, b, c, r, mode="e4m3")
        assert not emulated.TILE_SUM_EXACT
    per_board = (lib[0] - exact[0]).abs().reshape(64, -1).amax(1)
    assert per_board.median() < 1e-4                      # most boards: no flip, fp32 noise only
    assert 0.5 < (per_board <= 2e-2).float().mean() < 1.0  # some boards do flip ...
    assert 2e-2 < per_board.max() < 0.3                    # ... and then move by about 0.1


def test_teacher_forcing_entry_points_compose():
    # running layers [0,3) then [3,8) from the recorded residual stream is the whole forward
    sd, b, c, r = _golden_net()
    with torch.no_grad():
        taps = {}
        full = emulated.forward(sd, b, c, r, mode="e4m3", taps=taps)
        tail = emulated.forward(sd, b, c, r, mode="e4m3", x_in=taps["resid"][2], layer_begin=3)
    assert (full[0] == tail[0]).all() and (full[2] == tail[2]).all()


def test_packed_e4m3_blobs_have_the_layout_the_header_states():
    torch.manual_seed(1)
    net = BrokefishNet().eval()
    net.randomise_layers_(seed=2)
    sd = {k: v.detach() for k, v in net.state_dict().items()}
    stride = 5120
    ws, fp = hip_impl.pack_network(sd, 8, 256, 1024, 1, layer_stride=stride, fmt="e4m3")
    ws8, fp8 = hip_impl.pack_network(sd, 8, 256, 1024, 1, layer_stride=stride, fmt="int8")
    assert ws.size == ws8.size and fp.size == fp8.size
    # scale table of layer 2: 6 qkv + 2 out + 8 ffn1 + 2x4 ffn2 entries after the wsum block
    o_sw = 9 * 256 + 1024 + 4 * 256
    w2 = sd["encoder.layers.2.linear2.weight"]
    _, s2 = hip_impl.quantise_weights_e4m3(w2)
    assert (fp[2 * stride + o_sw + 16:2 * stride + o_sw + 24] == s2.reshape(-1)).all()
    assert (fp[2 * stride + o_sw - 1024:2 * stride + o_sw] == 0).all()          # no offset correction
    _, s2i = hip_impl.quantise_weights_int8(w2)
    assert (fp8[2 * stride + o_sw + 16:2 * stride + o_sw + 24] == np.repeat(s2i, 4)).all()
    # first block of layer 0: Q rows of head 0, fragment 0, lane 0 holds row 0, columns ch(r, 0)
    qb, _ = hip_impl.quantise_weights_e4m3(sd["encoder.layers.0.self_attn.in_proj_weight"])
    cols = [8 * (r // 4) + r % 4 for r in range(16)]
    assert (ws[:16] == qb[0, cols]).all()
