"""The kernels' row quantisers on their own (C-ABI ``bf_quant_probe``), against the reference's
quantiser arithmetic on the host: ``q = clamp(round_half_even(x / s))`` with ``x / s`` a true fp32
division (reference brokefish/nn/quant.py:246-260; device unit tests csrc/tests/tint8.cu:39-61 for
the ties and saturation, :190-227 for formula inputs).  The kernels build the quotient from a
reciprocal and two fused corrections, round by adding 1.5 * 2^23 with a byte-select add (signed) or
with v_cvt_pk_u8_f32 (unsigned, the ReLU being its saturation at 0), and convert to e4m3 with the
hardware's OCP conversion: each must give the byte the plain formula gives, ties included.
"""
import numpy as np
import pytest
import torch

from brokefish_amd import hip_impl

pytestmark = pytest.mark.gpu


def _run(x: np.ndarray, scale: float, mode: str) -> np.ndarray:
    pad = (-len(x)) % 4
    xt = torch.from_numpy(np.concatenate([x, np.zeros(pad, np.float32)]).astype(np.float32)).cuda()
    return hip_impl.quant_probe(xt, scale, mode).cpu().numpy()[:len(x)]


def _values(scale: np.float32, qmax: int, seed: int) -> np.ndarray:
    """Every tie k + 1/2 (exactly representable after the division where the scale is a power of
    two, and the nearest floats on either side of it otherwise), the integers, the ends of the
    range, and two million random values across it."""
    g = np.random.default_rng(seed)
    k = np.arange(-qmax - 1, qmax + 1, dtype=np.float64)
    ties = ((k + 0.5) * np.float64(scale)).astype(np.float32)
    near = np.concatenate([np.nextafter(ties, np.float32(np.inf)), np.nextafter(ties, np.float32(-np.inf)), ties])
    ints = (k * np.float64(scale)).astype(np.float32)
    rnd = (g.uniform(-qmax, qmax, 2_000_000) * np.float64(scale)).astype(np.float32)
    fine = (g.uniform(-2, 2, 200_000) * np.float64(scale)).astype(np.float32)
    return np.concatenate([near, ints, rnd, fine, np.array([0.0, -0.0, qmax * scale, -qmax * scale], np.float32)])


@pytest.mark.parametrize("scale", [1.0, 0.5, 0.0123, 3.7e-3, 127.0, 1.0 / 127.0, 2.0 ** -20])
def test_signed_quantiser_equals_division_and_round_half_even(scale):
    s = np.float32(scale)
    x = _values(s, 127, 1)
    x = x[np.abs(x / s) <= 127.0]                      # the row scale guarantees this range in the kernels
    want = np.rint(x / s).astype(np.int32)             # fp32 division (IEEE), then round half to even
    got = _run(x, float(s), "s8").view(np.int8).astype(np.int32)
    assert (got == want).all(), (x[got != want][:5], got[got != want][:5], want[got != want][:5])
    assert {-127, 0, 127} <= set(want.tolist())


@pytest.mark.parametrize("scale", [1.0, 0.25, 0.0123, 2.9e-3, 255.0, 1.0 / 255.0])
def test_unsigned_quantiser_folds_the_relu_into_its_saturation(scale):
    s = np.float32(scale)
    x = _values(s, 255, 2)
    x = x[x / s <= 255.0]
    want = np.clip(np.rint(np.maximum(x, np.float32(0)) / s), 0, 255).astype(np.int32)
    got = _run(x, float(s), "u8_relu").astype(np.int32)
    assert (got == want).all(), (x[got != want][:5], got[got != want][:5], want[got != want][:5])
    assert (got[x < 0] == 0).all() and got.max() == 255
    # the reference's own tie cases (csrc/tests/tint8.cu:59-61): .5 goes to the even neighbour
    ties = np.array([0.5, 1.5, 2.5, 3.5, 126.5, 127.5, 253.5, 254.5], np.float32)
    assert _run(ties, 1.0, "u8_relu").tolist() == [0, 2, 2, 4, 126, 128, 254, 254]
    assert _run(np.array([-0.5, -1.5, 0.5, 1.5, 2.5, -2.5, 126.5, -126.5], np.float32), 1.0, "s8").view(np.int8).tolist() == \
        [0, -2, 0, 2, 2, -2, 126, -126]


@pytest.mark.parametrize("scale", [1.0, 0.37, 1.0 / 8.0])
def test_e4m3_quantiser_equals_the_torch_cast(scale):
    s = np.float32(scale)
    g = np.random.default_rng(3)
    x = np.concatenate([(g.uniform(-9, 9, 1_000_000) * np.float64(s)).astype(np.float32),
                        (g.uniform(-500, 500, 100_000) * np.float64(s)).astype(np.float32),       # beyond the format's range: clamped
                        (g.uniform(-0.02, 0.02, 100_000) * np.float64(s)).astype(np.float32)])    # subnormal codes
    q = torch.from_numpy(x) / torch.tensor(s)
    want = q.clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = _run(x, float(s), "e4m3")
    # -0 and +0 are the same number; everything else must be the same code
    same = (got == want) | (((got & 0x7F) == 0) & ((want & 0x7F) == 0))
    assert same.all(), (x[~same][:5], got[~same][:5], want[~same][:5])


def test_probe_rejects_bad_arguments():
    x = torch.zeros(8, device="cuda")
    with pytest.raises(ValueError):
        hip_impl.quant_probe(x[:6], 1.0, "s8")
    with pytest.raises(ValueError):
        hip_impl.quant_probe(x, 1.0, "u4")
    with pytest.raises(RuntimeError):
        hip_impl.quant_probe(x, 0.0, "s8")
