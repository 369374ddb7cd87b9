"""NF4 oracle: the code book re-derived from its published construction (normal quantiles), closed
forms and round trips.  Its parity with the bitsandbytes library itself stays unpinned: the library
is not available and the reference holds no NF4 vectors."""
import numpy as np
import torch

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


def test_nf4_table_is_the_normal_quantile_construction():
    """The 16 NF4 values are not free constants: they are quantiles of N(0, 1) at evenly spaced probabilities
    (8 on the positive side from 0.9677083 down to 0.5 exclusive, 7 on the negative side), an exact 0, sorted
    and divided by the largest (QLoRA, appendix E; bitsandbytes `create_normal_map(offset=0.9677083)`).  A typo
    in any entry of the oracle's table (and of the product's, which must equal it) fails this."""
    from scipy.stats import norm

    offset = 0.9677083
    pos = norm.ppf(torch.linspace(offset, 0.5, 9)[:-1].numpy())
    neg = -norm.ppf(torch.linspace(offset, 0.5, 8)[:-1].numpy())
    table = torch.tensor(np.concatenate([pos, [0.0], neg])).sort().values
    table = (table / table.max()).to(torch.float32).numpy()
    assert table.shape == (16,)
    assert np.array_equal(table, nf4.NF4), np.abs(table - nf4.NF4).max()
    # asymmetric on purpose: 7 negative and 8 positive levels around an exact zero
    assert (nf4.NF4 < 0).sum() == 7 and (nf4.NF4 > 0).sum() == 8
    from fms_acceleration_peft.nf4 import NF4_CODE

    assert np.array_equal(np.asarray(NF4_CODE, np.float32), nf4.NF4)


def test_dynamic_map_known_entries():
    """Entries of the signed 8-bit dynamic map that follow from its construction (7 exponent levels, level i holds
    the 2**i midpoints of linspace(0.1, 1, 2**i + 1) scaled by 10**(i - 6), both signs, then 0 and 1)."""
    m = nf4.dynamic_map_8bit()
    assert np.unique(m).size == 256                     # 2 * (1 + 2 + ... + 64) + 2 distinct values
    assert m[0] == np.float32(-(1.0 - 0.9 / 128))       # last midpoint of level 6: -(1 - 0.9 / 64 / 2)
    assert m[m > 0][0] == np.float32(0.55e-6)           # level 0: the one midpoint of [0.1, 1] times 1e-6
    assert m[m > 0][1] == np.float32(0.325e-5) and m[m > 0][2] == np.float32(0.775e-5)  # level 1
    assert m[-2] == np.float32(1.0 - 0.9 / 128) and m[-1] == 1.0
    assert (m < 0).sum() == 127 and (m > 0).sum() == 128
    assert np.array_equal(np.sort(-m[m < 0]), m[(m > 0) & (m < 1)])  # symmetric apart from the extra 1.0
    from fms_acceleration_peft.nf4 import dynamic_map_8bit

    assert np.array_equal(dynamic_map_8bit().numpy(), m)
