"""Pins the CPU oracle's GPTQ layout / quantiser / dequantisation by checks that do not restate
its formulas: brute-force scalar loops, round trips, algebraic identities and invariants."""
import numpy as np
import pytest
import torch

from oracle import gptq


def test_pack_layout_bit_by_bit():
    """Scalar loop over every nibble of a tiny matrix: row 8*i+j of q sits in bits 4j..4j+3 of
    word [i, n]; column 8*i+j of z sits in bits 4j..4j+3 of word [g, i]."""
    rng = np.random.default_rng(0)
    q = rng.integers(0, 16, size=(32, 32))
    qw = gptq.pack_rows(q).view(np.uint32)
    assert qw.shape == (4, 32) and qw.dtype == np.uint32
    for k in range(32):
        for n in range(32):
            assert (int(qw[k // 8, n]) >> (4 * (k % 8))) & 15 == q[k, n]
    z = rng.integers(0, 16, size=(2, 32))
    qz = gptq.pack_cols(z).view(np.uint32)
    assert qz.shape == (2, 4)
    for g in range(2):
        for n in range(32):
            assert (int(qz[g, n // 8]) >> (4 * (n % 8))) & 15 == z[g, n]


def test_pack_known_word():
    """Known-answer word: rows 0..7 holding 0..7 pack to 0x76543210; all 15 packs to -1 (int32)."""
    q = np.tile(np.arange(8)[:, None], (1, 32))
    assert gptq.pack_rows(q).view(np.uint32)[0, 0] == 0x76543210
    assert gptq.pack_rows(np.full((8, 32), 15))[0, 0] == -1
    z = np.tile(np.arange(8)[None, :], (1, 4))
    assert gptq.pack_cols(z).view(np.uint32)[0, 0] == 0x76543210


@pytest.mark.parametrize("K,N", [(32, 32), (256, 96), (128, 160)])
def test_pack_unpack_round_trip(K, N):
    rng = np.random.default_rng(K + N)
    q = rng.integers(0, 16, size=(K, N))
    assert np.array_equal(gptq.unpack_rows(gptq.pack_rows(q)), q)
    z = rng.integers(0, 16, size=(K // 32, N))
    assert np.array_equal(gptq.unpack_cols(gptq.pack_cols(z)), z)


def test_dequant_scalar_loop():
    """Element-by-element python arithmetic on K = N = 32 with a shuffled g_idx."""
    rng = np.random.default_rng(1)
    K = N = 32
    G = 4
    q = rng.integers(0, 16, size=(K, N))
    z = rng.integers(0, 16, size=(G, N))
    s = rng.random((G, N)).astype(np.float16) * np.float16(0.02) + np.float16(0.001)
    g_idx = rng.permutation(np.repeat(np.arange(G), K // G)).astype(np.int32)
    W = gptq.dequant(gptq.pack_rows(q), s, gptq.pack_cols(z), g_idx, out="fp32").numpy()
    for k in range(K):
        for n in range(N):
            g = g_idx[k]
            assert W[k, n] == np.float32(float(s[g, n]) * (int(q[k, n]) - int(z[g, n])))


def test_dequant_fp32_product_is_exact():
    """fp16 scale (11 significant bits) times an integer in [-16, 15] fits fp32: the float64 and the
    float32 evaluations agree bit for bit, so fp16/bf16 outputs carry exactly one rounding."""
    rng = np.random.default_rng(2)
    s = rng.random((8, 64)).astype(np.float16)
    d = rng.integers(-16, 16, size=(8, 64))
    exact = s.astype(np.float64) * d
    assert np.array_equal(exact, (s.astype(np.float32) * d.astype(np.float32)).astype(np.float64))


def test_v1_v2_zero_point_identity():
    """dequant(v1 zeros, zero_offset=1) == dequant(v1 zeros + 0x11111111, zero_offset=0): the
    conversion the local loader applies to AutoGPTQ v1 checkpoints."""
    rng = np.random.default_rng(3)
    K, N, G = 128, 64, 2
    qw = gptq.pack_rows(rng.integers(0, 16, size=(K, N)))
    z_v1 = rng.integers(0, 15, size=(G, N))  # stored zero - 1, so the true zero is <= 15
    s = (rng.random((G, N)) * 0.02 + 0.001).astype(np.float16)
    qz_v1 = gptq.pack_cols(z_v1)
    qz_v2 = (qz_v1.view(np.uint32) + np.uint32(0x11111111)).view(np.int32)
    a = gptq.dequant(qw, s, qz_v1, None, 64, zero_offset=1, out="fp16")
    b = gptq.dequant(qw, s, qz_v2, None, 64, zero_offset=0, out="fp16")
    assert torch.equal(a, b)
    assert np.array_equal(gptq.to_v1_zeros(qz_v2), qz_v1)


def test_identity_g_idx_and_negative_wrap():
    rng = np.random.default_rng(4)
    K, N, gs = 256, 32, 64
    buf = gptq.quantize_and_pack(rng.standard_normal((N, K)).astype(np.float32) * 0.02, gs)
    assert np.array_equal(buf["g_idx"], np.arange(K) // gs)
    a = gptq.dequant(buf["qweight"], buf["scales"], buf["qzeros"], None, gs, out="fp32")
    b = gptq.dequant(buf["qweight"], buf["scales"], buf["qzeros"], buf["g_idx"], out="fp32")
    assert torch.equal(a, b)
    neg = buf["g_idx"].copy()
    neg[neg == 3] = -1  # group index -1 wraps to the last group
    assert torch.equal(gptq.dequant(buf["qweight"], buf["scales"], buf["qzeros"], neg, out="fp32"), b)


def test_act_order_joint_permutation_invariance():
    """Permuting the rows of q together with g_idx permutes the rows of W and nothing else."""
    rng = np.random.default_rng(5)
    K, N, gs = 256, 64, 64
    W0 = rng.standard_normal((N, K)).astype(np.float32) * 0.02
    g_idx = gptq.act_order_g_idx(K, gs, seed=7)
    assert all((g_idx == g).sum() == gs for g in range(K // gs))
    q, s, z, _ = gptq.rtn_quantize(W0, gs, g_idx=g_idx)
    W = gptq.dequant(gptq.pack_rows(q), s, gptq.pack_cols(z), g_idx, out="fp32")
    perm = rng.permutation(K)
    Wp = gptq.dequant(gptq.pack_rows(q[perm]), s, gptq.pack_cols(z), g_idx[perm], out="fp32")
    assert torch.equal(Wp, W[perm])
    # y = x W is invariant under the joint permutation of x's columns and W's rows
    x = torch.from_numpy(rng.standard_normal((8, K))).float()
    torch.testing.assert_close(x[:, perm] @ Wp, x @ W, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("sym", [False, True])
def test_rtn_invariants(sym):
    """zero in [0, 15]; q in [0, 15]; inside the clamp range |W - deq| <= scale/2 (+fp16 scale error);
    an all-zero group falls back to (-1, 1); symmetric mode centres the zero at 8."""
    rng = np.random.default_rng(6)
    N, K, gs = 48, 256, 128
    W = rng.standard_normal((N, K)).astype(np.float32) * 0.02
    W[5, :gs] = 0.0
    q, s, z, g = gptq.rtn_quantize(W, gs, sym=sym)
    assert q.min() >= 0 and q.max() <= 15 and z.min() >= 0 and z.max() <= 16
    assert s.dtype == np.float16 and np.all(s > 0)
    assert abs(float(s[0, 5]) - 2.0 / 15) < 1e-3  # dead group: (xmax - xmin)/15 with (-1, 1)
    if sym:
        assert np.all(z == 8)
    deq = gptq.dequant_f64(gptq.pack_rows(q), s, gptq.pack_cols(np.minimum(z, 15)), g)
    err = np.abs(deq - W.T.astype(np.float64))
    inside = (q > 0) & (q < 15) & (z[g] <= 15)
    bound = 0.5 * s.astype(np.float64)[g] * (1 + 2e-3) + 1e-6 + 16 * 2e-3 * s.astype(np.float64)[g]
    assert np.all(err[inside] <= bound[inside])


def test_torch_dequant_restatement_agrees():
    """The shift/mask/gather formulation used by the CPU baseline equals the exact one."""
    rng = np.random.default_rng(8)
    N, K, gs = 64, 256, 64
    g_idx = gptq.act_order_g_idx(K, gs, seed=1)
    buf = gptq.quantize_and_pack(rng.standard_normal((N, K)).astype(np.float32) * 0.02, gs, g_idx=g_idx)
    a = gptq.dequant(buf["qweight"], buf["scales"], buf["qzeros"], buf["g_idx"], out="fp32")
    b = gptq.dequant_torch(buf["qweight"], buf["scales"], buf["qzeros"], buf["g_idx"])
    assert torch.equal(a, b)
    c = gptq.dequant_torch(buf["qweight"], buf["scales"], gptq.to_v1_zeros(buf["qzeros"]), buf["g_idx"], zero_offset=1)
    assert torch.equal(a, c)


def test_product_quantiser_matches_oracle():
    """The torch quantiser shipped with the package (used to build synthetic checkpoints) against
    the numpy oracle, identity and act-order."""
    from fms_acceleration_peft.quantizer import rtn_quantize

    g = torch.Generator().manual_seed(0)
    W = torch.randn(96, 256, generator=g) * 0.02
    for act_order in (False, True):
        gi = gptq.act_order_g_idx(256, 64, seed=1) if act_order else None
        a = rtn_quantize(W, 4, 64, g_idx=None if gi is None else torch.from_numpy(gi))
        b = gptq.quantize_and_pack(W.numpy(), 64, g_idx=gi)
        for k in ("qweight", "qzeros", "scales", "g_idx"):
            assert np.array_equal(a[k].numpy(), b[k]), k
