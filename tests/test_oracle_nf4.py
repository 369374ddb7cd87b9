"""NF4 oracle: closed forms and round trips (its parity with bitsandbytes itself is unpinned: the
library is not available and the reference holds no NF4 vectors)."""
import numpy as np

from oracle import nf4


def test_codebook_shape_and_order():
    assert nf4.NF4.size == 16 and nf4.NF4[0] == -1 and nf4.NF4[7] == 0 and nf4.NF4[15] == 1
    assert np.all(np.diff(nf4.NF4) > 0)
    m = nf4.dynamic_map_8bit()
    assert m.size == 256 and np.all(np.diff(m) >= 0) and m[-1] == 1.0 and (m == 0).sum() == 1
    assert m.min() > -1.0 and abs(m.min() + 0.9929688) < 1e-3  # largest negative midpoint


def test_nibble_order_high_first():
    """A weight whose first element is the block maximum and second is zero packs to 0xF7."""
    W = np.zeros((1, 64), np.float32)
    W[0, 0], W[0, 1], W[0, 2] = 2.0, 0.0, -2.0
    q = nf4.quantize(W)
    assert q["packed"][0, 0] == 0xF7 and q["packed"][1, 0] >> 4 == 0x0
    d = nf4.dequant(q, "fp32").numpy()
    assert abs(d[0, 0] - 2.0) < 2e-2 and d[0, 1] == 0.0 and abs(d[0, 2] + 2.0) < 2e-2


def test_round_trip_error_bounds():
    rng = np.random.default_rng(0)
    W = (rng.standard_normal((96, 512)) * 0.02).astype(np.float32)
    q = nf4.quantize(W)
    assert q["packed"].shape == (96 * 512 // 2, 1) and q["absmax_q"].size == 96 * 512 // 64
    absmax_true = np.abs(W.reshape(-1, 64)).max(axis=1)
    absmax = nf4.dequant_absmax(q)
    # 8-bit double quantisation of (absmax - mean): error small relative to the spread
    assert np.abs(absmax - absmax_true).max() < 0.05 * (absmax_true.max() - absmax_true.min()) + 1e-6
    d = nf4.dequant(q, "fp32").numpy()
    half_gap = np.max(np.diff(nf4.NF4)) / 2
    bound = absmax.repeat(64).reshape(W.shape) * half_gap + np.abs(absmax - absmax_true).repeat(64).reshape(W.shape) + 1e-6
    assert np.all(np.abs(d - W) <= bound)


def test_exact_codes_are_fixed_points():
    """Weights that are exactly code * absmax with absmax representable by the double quantisation
    (every block has the same absmax, so absmax - offset == 0) survive quantise->dequantise exactly."""
    rng = np.random.default_rng(1)
    idx = rng.integers(0, 16, size=(4, 128))
    idx[:, 0] = 15
    idx[:, 64] = 15
    W = (nf4.NF4[idx] * np.float32(0.5)).astype(np.float32)
    q = nf4.quantize(W)
    assert np.array_equal(nf4.dequant(q, "fp32").numpy(), W)
