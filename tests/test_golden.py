"""The committed vectors (tests/golden/hot_path_small.npz) against the CPU oracle -- and, where the
value is a closed form of the bit layout, against plain loops that do not go through the oracle."""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURE = os.path.join(HERE, "golden", "hot_path_small.npz")


@pytest.fixture(scope="module")
def gold():
    with np.load(FIXTURE) as z:  # allow_pickle stays False
        return {k: z[k] for k in z.files}


def test_oracle_reproduces_every_vector(gold):
    sys.path.insert(0, os.path.join(HERE, "golden"))
    import make_fixtures

    fresh = make_fixtures.build()
    assert set(fresh) == set(gold)
    for name, want in gold.items():
        got = np.asarray(fresh[name])
        assert got.shape == want.shape and got.dtype == want.dtype, name
        if want.dtype.kind in "iu":
            assert np.array_equal(got, want), name  # packed words, indices, 16-bit patterns
        else:
            assert np.allclose(got, want, rtol=1e-9, atol=1e-12), name  # fp64 sums may be reordered by the BLAS


def _rne_bf16_bits(x: float) -> int:
    """float -> bf16 bit pattern, round to nearest even, from the fp32 encoding."""
    u = int(np.float32(x).view(np.uint32))
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF


@pytest.mark.parametrize("tag", ["deq", "deq_act"])
def test_dequantised_weights_from_the_bit_layout(gold, tag):
    """W[k, n] = scale[g, n] * (nibble k%8 of qweight[k//8, n] - nibble n%8 of qzeros[g, n//8]), g = g_idx[k]
    (qlinear_tritonv2.py:132-165 for the packing, kernels.py:72-116 for the indexing), one rounding."""
    qw, qz, sc, gi = (gold[f"{tag}.{k}"] for k in ("qweight", "qzeros", "scales", "g_idx"))
    K, N = qw.shape[0] * 8, qw.shape[1]
    rng = np.random.default_rng(0)
    for k, n in zip(rng.integers(0, K, 400), rng.integers(0, N, 400)):
        q = (int(qw[k // 8, n]) >> (4 * (k % 8))) & 15
        g = int(gi[k])
        z = (int(qz[g, n // 8]) >> (4 * (n % 8))) & 15
        value = float(sc[g, n]) * (q - z)  # exact in binary64 (11-bit x 5-bit)
        assert int(np.float16(value).view(np.uint16)) == int(gold[f"{tag}.W_fp16"][k, n])
        assert _rne_bf16_bits(value) == int(gold[f"{tag}.W_bf16"][k, n])
    if tag == "deq_act":
        assert not np.array_equal(gi, np.arange(K) // 64) and np.array_equal(np.bincount(gi), np.full(K // 64, 64))


def test_v1_zero_points_are_the_same_weights(gold):
    """The v1 checkpoint format stores zero - 1 in every nibble (gptqmodel/utils/model.py:230-231)."""
    v1, v2 = gold["deq.qzeros_v1"].view(np.uint32), gold["deq.qzeros"].view(np.uint32)
    for j in range(8):
        assert np.array_equal(((v1 >> (4 * j)) & 15) + 1, (v2 >> (4 * j)) & 15)


def test_nf4_weights_from_the_bit_layout(gold):
    """Element 2i sits in the high nibble of byte i; absmax = code2[absmax_q] * absmax2[block // 256] + offset."""
    nf4 = [-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635, -0.18477343022823334,
           -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725, 0.24611230194568634, 0.33791524171829224,
           0.44070982933044434, 0.5626170039176941, 0.7229568362236023, 1.0]
    packed = gold["nf4.packed"].reshape(-1)
    bs, bs2 = int(gold["nf4.blocksize"]), int(gold["nf4.blocksize2"])
    want = gold["nf4.W_bf16"].reshape(-1)
    rng = np.random.default_rng(1)
    for i in rng.integers(0, want.size, 400):
        nib = (int(packed[i // 2]) >> 4) if i % 2 == 0 else (int(packed[i // 2]) & 15)
        blk = i // bs
        absmax = np.float32(np.float32(gold["nf4.code2"][gold["nf4.absmax_q"][blk]]) * np.float32(gold["nf4.absmax2"][blk // bs2])) \
            + np.float32(gold["nf4.offset"])
        assert _rne_bf16_bits(float(np.float32(nf4[nib]) * np.float32(absmax))) == int(want[i])


def test_swiglu_vectors_follow_the_rounding_points(gold):
    """f = bf16(e * sigmoid(e)), h = bf16(f * g), d_g = bf16(dh * f), d_e = bf16(bf16(dh * g) * s (1 + e (1 - s)))
    (unsloth_lora/swiglu.py:26-33, 65-83), restated in binary64 + explicit roundings.  A binary64 sigmoid can
    differ from the fp32 one in the last place, which moves a rounding in rare cases: at most one step of
    the 16-bit result, and on under 1 % of the entries."""
    def up(b):
        return (b.astype(np.uint32) << 16).view(np.float32).astype(np.float64)

    def rnd(x):
        return up(np.vectorize(_rne_bf16_bits, otypes=[np.uint32])(x).astype(np.uint16))

    e, g, dh = (up(gold[f"swiglu.bf16.{k}"]) for k in ("e", "g", "dh"))
    s = 1.0 / (1.0 + np.exp(-e))
    f = rnd(e * s)
    for name, mine in (("h", rnd(f * g)), ("d_g", rnd(dh * f)), ("d_e", rnd(rnd(dh * g) * s * (1.0 + e * (1.0 - s))))):
        want = up(gold[f"swiglu.bf16.{name}"])
        assert np.mean(mine == want) > 0.99, name
        assert np.all(np.abs(mine - want) <= np.abs(want) * 2.0 ** -7 + 1e-30), name


def test_lora_vectors_satisfy_the_closed_forms(gold):
    """dB = s dY^T (X A^T) and dA = s (dY B)^T X (fast_lora.py:822-825), evaluated here with numpy on the
    stored inputs -- the vectors themselves came from autograd of the unfused graph."""
    def up(b):
        return (b.astype(np.uint32) << 16).view(np.float32).astype(np.float64)

    x, dy, A, B, s = up(gold["lora_w.x"]), up(gold["lora_w.dy"]), up(gold["lora_w.A"]), up(gold["lora_w.B"]), float(gold["lora_w.s"])
    assert np.allclose(gold["lora_w.dB"], s * dy.T @ (x @ A.T), rtol=1e-9, atol=1e-12)
    assert np.allclose(gold["lora_w.dA"], s * (dy @ B).T @ x, rtol=1e-9, atol=1e-12)
    # y and dX need the dense weight: unpacked here with numpy shifts, independently of the oracle
    qw, qz, sc, gi = (gold[f"lora_w.{k}"] for k in ("qweight", "qzeros", "scales", "g_idx"))
    K, N = qw.shape[0] * 8, qw.shape[1]
    k, n = np.arange(K)[:, None], np.arange(N)[None, :]
    q = (qw.view(np.uint32)[k // 8, n] >> (4 * (k % 8)).astype(np.uint32)) & 15
    z = (qz.view(np.uint32)[gi[k], n // 8] >> (4 * (n % 8)).astype(np.uint32)) & 15
    W = sc.astype(np.float64)[gi[k], n] * (q.astype(np.float64) - z.astype(np.float64))
    assert np.allclose(gold["lora_w.y"], x @ W + s * (x @ A.T) @ B.T, rtol=1e-9, atol=1e-12)
    assert np.allclose(gold["lora_w.dx"], dy @ W.T + s * (dy @ B) @ A, rtol=1e-9, atol=1e-12)
