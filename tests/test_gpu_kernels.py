"""GPU parity tests of the C-ABI kernels against the CPU oracle (run on the MI355X box)."""
import pytest
import torch

from oracle import gptq as ogptq
from oracle import lora as olora
from tests.helpers import make_gptq, randn

pytestmark = pytest.mark.gpu

TOL = 1e-2  # max |out - ref| / max |ref| against the fp32 oracle, per tensor


def dev(t):
    return t.cuda()


def gweight(w, identity=True, interleaved=False):
    import fmsa_hip

    t = w.get("dev")  # the C struct holds raw pointers: one device copy per weight, kept alive by the dict
    if t is None:
        t = {k: dev(v) for k, v in w["t"].items()}
        w["dev"] = t
    if interleaved:  # the forward kernel's packed-half unpack (fp16 activations) reads this copy
        if "qweight_il" not in t:
            t["qweight_il"] = fmsa_hip.gptq_interleave(t["qweight"])
        return fmsa_hip.make_weight(t["qweight_il"], t["scales"], t["qzeros"], None, w["group_size"], w["zero_offset"],
                                    nibble_order=1)
    return fmsa_hip.make_weight(t["qweight"], t["scales"], t["qzeros"], None if identity else t["g_idx"],
                                w["group_size"], w["zero_offset"])


@pytest.mark.parametrize("K,N,gs", [(256, 256, 128), (2048, 2048, 128), (96, 160, 32), (512, 1024, 64)])
@pytest.mark.parametrize("act_order", [False, True])
@pytest.mark.parametrize("v1", [False, True])
def test_dequant_bit_exact(K, N, gs, act_order, v1):
    import fmsa_hip

    w = make_gptq(K, N, gs, seed=K + N, act_order=act_order, v1=v1)
    t = {k: dev(v) for k, v in w["t"].items()}
    for name, dt in (("fp16", torch.float16), ("bf16", torch.bfloat16), ("fp32", torch.float32)):
        ref = ogptq.dequant(w["np"]["qweight"], w["np"]["scales"], w["np"]["qzeros"], w["np"]["g_idx"],
                            zero_offset=w["zero_offset"], out=name)
        out = fmsa_hip.gptq_dequant(t["qweight"], t["scales"], t["qzeros"], t["g_idx"], w["group_size"],
                                    w["zero_offset"], dt).cpu()
        assert torch.equal(out.view(torch.int16 if dt != torch.float32 else torch.int32),
                           ref.view(torch.int16 if dt != torch.float32 else torch.int32)), name
        if not act_order:  # NULL g_idx means k // group_size
            out2 = fmsa_hip.gptq_dequant(t["qweight"], t["scales"], t["qzeros"], None, w["group_size"],
                                         w["zero_offset"], dt).cpu()
            assert torch.equal(out2, out)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,C,r", [(512, 2048, 16), (200, 4096, 8), (64, 1056, 64), (33, 96, 24), (300, 2048, 96), (8192, 1024, 128)])
def test_lora_down(M, C, r, dtype):
    import fmsa_hip

    x = randn((M, C), 2, dtype)
    wd = randn((r, C), 1, dtype, 0.05)
    ref = x.float() @ wd.float().t()
    out = fmsa_hip.lora_down(dev(x), dev(wd)).cpu()
    assert olora.max_rel_err(out, ref) < 5e-3


@pytest.mark.parametrize("M,C", [(100, 2048), (4096, 8192), (33, 28672), (7, 40000), (64, 1032)])
def test_permute_cols(M, C):
    """Column gather / scatter of an activation matrix (rows staged through LDS up to 64 KB per row, the
    direct kernel beyond): against torch indexing, bit for bit, for a row-strided input too."""
    import fmsa_hip

    gen = torch.Generator().manual_seed(M + C)
    perm = torch.randperm(C, generator=gen).to(torch.int32).cuda()
    wide = dev(randn((M, C + 16), 3, torch.bfloat16))
    for x in (wide[:, :C].contiguous(), wide[:, 8 : 8 + C]):
        g = fmsa_hip.permute_cols(x, perm, gather=True)
        assert torch.equal(g, x[:, perm.long()])
        sc = fmsa_hip.permute_cols(x, perm, gather=False)
        ref = torch.empty_like(sc)
        ref[:, perm.long()] = x
        assert torch.equal(sc, ref)
        assert torch.equal(fmsa_hip.permute_cols(g, perm, gather=False), x)  # scatter undoes gather


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,C,r", [(4096, 28672, 64), (4100, 8192, 32), (8192, 4096, 96), (8200, 2048, 128), (4096, 8200, 120), (8192, 8200, 16), (8200, 14336, 32), (8192, 2048, 48), (8222, 9000, 64), (8192, 4096, 24)])
def test_lora_down_many_tokens(M, C, r, dtype):
    """From 8192 tokens on, long rows / stacked ranks take the kernel that stages X through LDS: ragged
    token and column counts (last workgroup of 8 or 30 rows, last 512-column stage of 8 or 296 columns),
    X as a column slice of a wider matrix and the output as a column slice of a stacked one."""
    import fmsa_hip

    xw = dev(randn((M, C + 24), 12, dtype))
    x = xw[:, 8 : 8 + C]  # row stride C + 24, base 16 bytes into the row
    wd = dev(randn((r, C), 13, dtype, 0.05))
    ref = x.float() @ wd.float().t()
    out_cat = torch.full((M, r + 16), 7.0, dtype=dtype, device=x.device)
    out = fmsa_hip.lora_down(x, wd, out=out_cat[:, 8 : 8 + r])
    assert olora.max_rel_err(out.cpu(), ref.cpu()) < 5e-3
    assert torch.all(out_cat[:, :8] == 7.0) and torch.all(out_cat[:, 8 + r :] == 7.0)
    assert torch.equal(fmsa_hip.lora_down(x, wd), out)  # run-to-run bit-stable, whatever the output stride


@pytest.mark.parametrize("M,C,r", [(4096, 8192, 64), (2048, 4096, 32), (2100, 2048, 128), (16384, 14336, 32)])
def test_lora_down_with_and_without_workspace(M, C, r):
    """From rank 32 on fmsa_lora_down_ws takes 64-128 tokens per workgroup and splits the columns over workgroups whose
    sums meet in the workspace; without a workspace, or with an output the reduce pass cannot store into four ranks at a
    time, it runs as fmsa_lora_down does.  Every route against the fp32 product; each is bit-stable run to run."""
    import ctypes

    import fmsa_hip

    lib = fmsa_hip.lib()
    dtype = torch.bfloat16
    x = dev(randn((M, C), 21, dtype))
    wd = dev(randn((r, C), 22, dtype, 0.05))
    ref = (x.float() @ wd.float().t()).cpu()
    need = lib.fmsa_lora_down_workspace(M, C, r)
    assert (need > 0) == (M < 16384)  # 16384 tokens at rank 32: 256 workgroups of 64 tokens, no column split
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=x.device)

    def run(out, workspace, nbytes):
        rc = lib.fmsa_lora_down_ws(x.data_ptr(), x.stride(0), wd.data_ptr(), M, C, r, fmsa_hip.act_enum(dtype), out.data_ptr(),
                                   out.stride(0), workspace, nbytes, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, rc
        return out

    with_ws = run(torch.empty(M, r, dtype=dtype, device=x.device), ws.data_ptr(), ws.numel())
    assert torch.equal(with_ws, run(torch.empty_like(with_ws), ws.data_ptr(), ws.numel()))
    without = run(torch.empty_like(with_ws), None, 0)
    plain = fmsa_hip.lora_down(x, wd)
    small = run(torch.empty_like(with_ws), ws.data_ptr(), max(need // 2, 1)) if need else without
    odd = torch.zeros(M, r + 6, dtype=dtype, device=x.device)  # rows 4 bytes off an 8-byte boundary, stride % 4 != 0
    run(odd[:, 2 : 2 + r], ws.data_ptr(), ws.numel())
    for out in (with_ws, without, plain, small, odd[:, 2 : 2 + r]):
        assert olora.max_rel_err(out.cpu(), ref) < 5e-3
    assert torch.equal(plain, with_ws)      # the binding brings the workspace
    assert torch.equal(small, without)      # too small a buffer is as good as none
    assert torch.all(odd[:, :2] == 0) and torch.all(odd[:, 2 + r :] == 0)
    if need:
        assert lib.fmsa_lora_down_ws(x.data_ptr(), x.stride(0), wd.data_ptr(), M, C, r, fmsa_hip.act_enum(dtype), with_ws.data_ptr(),
                                     with_ws.stride(0), ws.data_ptr() + 4, ws.numel() - 4, None) == -3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,C,r,tr", [(512, 2048, 16, False), (200, 1056, 8, True), (4096, 4096, 16, True), (96, 136, 24, False), (70, 4104, 64, True),
                                      (1000, 2048, 96, False), (333, 520, 128, True)])
def test_lora_grad(M, C, r, tr, dtype):
    import fmsa_hip

    L = randn((M, r), 5, dtype)
    R = randn((M, C), 6, dtype)
    ref = 0.5 * (L.float().t() @ R.float())
    if tr:
        ref = ref.t()
    out = fmsa_hip.lora_grad(dev(L), dev(R), 0.5, tr, torch.float32).cpu()
    assert out.shape == ref.shape
    assert olora.max_rel_err(out, ref) < 1e-4
    out2 = fmsa_hip.lora_grad(dev(L), dev(R), 0.5, tr, torch.float32).cpu()
    assert torch.equal(out, out2), "two-pass reduction must be run-to-run bit-stable"
    outb = fmsa_hip.lora_grad(dev(L), dev(R), 0.5, tr, dtype).cpu()
    assert olora.max_rel_err(outb, ref) < 5e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_lora_grad_batch_equals_separate_calls(dtype):
    """Jobs of different widths, ranks, layouts and output types in one launch: each result is bit
    for bit what fmsa_lora_grad gives for that job alone (checked against the fp32 product above).
    Ten jobs also cover the split into launches of at most eight."""
    import fmsa_hip

    M = 1111
    shapes = [(2048, 48, False, torch.float32), (2048, 16, True, dtype), (520, 16, True, torch.float32), (136, 8, False, dtype),
              (4104, 64, True, torch.float32), (1056, 96, False, torch.float32), (96, 24, True, dtype), (2048, 16, True, torch.float32),
              (520, 128, False, dtype), (8, 8, False, torch.float32)]
    jobs = []
    for i, (C, r, tr, od) in enumerate(shapes):
        Lfull = dev(randn((M, r + 8), 70 + i, dtype))  # a column slice: row stride > r
        jobs.append((Lfull[:, :r], dev(randn((M, C), 90 + i, dtype)), 0.5 + i, tr, od))
    outs = fmsa_hip.lora_grad_batch(jobs)
    assert len(outs) == len(jobs)
    for (L, R, scale, tr, od), out in zip(jobs, outs):
        single = fmsa_hip.lora_grad(L, R, scale, tr, od)
        assert out.dtype == od and out.shape == single.shape
        assert torch.equal(out, single)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_lora_grad_batch_with_T(dtype):
    """Jobs that also produce T = R @ Wt^T from the same pass over R: ragged token / column counts (last
    token tile of 23 rows, last column block of 8 columns), T written as a column slice of a stacked
    matrix, ranks 8 / 16 / 32, next to a job without T.  T against the fp32 product and against
    lora_down (same rounding point, other order of the sums); the gradients bit for bit as without T."""
    import fmsa_hip

    M = 2327
    shapes = [(4104, 16, True), (1056, 8, False), (136, 32, True), (2048, 16, True)]
    T_cat = torch.full((M, 80), 3.0, dtype=dtype, device="cuda")
    jobs, o = [], 0
    for i, (C, r, tr) in enumerate(shapes):
        L, R, Wt = dev(randn((M, r), 110 + i, dtype)), dev(randn((M, C), 120 + i, dtype)), dev(randn((r, C), 130 + i, dtype, 0.05))
        with_t = i != 1
        jobs.append((L, R, 0.5, tr, torch.float32) + ((Wt, T_cat[:, o : o + r]) if with_t else ()))
        o += r if with_t else 0
    outs = fmsa_hip.lora_grad_batch(jobs)
    assert torch.all(T_cat[:, o:] == 3.0)
    for job, out in zip(jobs, outs):
        L, R, scale, tr, od = job[:5]
        assert torch.equal(out, fmsa_hip.lora_grad(L, R, scale, tr, od))
        if len(job) > 5:
            Wt, T = job[5:]
            ref = R.float() @ Wt.float().t()
            assert olora.max_rel_err(T.float().cpu(), ref.cpu()) < 5e-3
            assert olora.max_rel_err(T.float().cpu(), fmsa_hip.lora_down(R, Wt).float().cpu()) < 5e-3
    T_first = T_cat.clone()
    fmsa_hip.lora_grad_batch(jobs)
    assert torch.equal(T_cat, T_first)  # run-to-run bit-stable


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_lora_pack_batch(dtype):
    """Five adapters of different shapes and parameter types in one call (two launches): every copy is
    the parameter rounded once to the activation type, A16 of the first three lands inside a stacked
    matrix."""
    import fmsa_hip

    shapes = [(16, 2048, 4096, torch.float32), (8, 2048, 1024, torch.float32), (24, 2048, 1024, torch.bfloat16),
              (64, 1056, 96, torch.float16), (16, 96, 14336, torch.float32)]
    A_cat = torch.zeros((48, 2048), dtype=dtype, device="cuda")
    adapters, o = [], 0
    for i, (r, K, N, pd) in enumerate(shapes):
        A = dev(randn((r, K), 30 + i, torch.float32)).to(pd)
        B = dev(randn((N, r), 40 + i, torch.float32)).to(pd)
        adapters.append((A, B, A_cat[o : o + r] if i < 3 else None))
        o += r if i < 3 else 0
    outs = fmsa_hip.lora_pack_batch(adapters, dtype)
    for (A, B, slot), (A16, At16, B16, Bt16) in zip(adapters, outs):
        assert torch.equal(A16, A.to(dtype)) and torch.equal(At16, A.to(dtype).t())
        assert torch.equal(B16, B.to(dtype)) and torch.equal(Bt16, B.to(dtype).t())
        assert slot is None or A16.data_ptr() == slot.data_ptr()
        single = fmsa_hip.lora_pack(A, B, dtype)
        assert all(torch.equal(x, y) for x, y in zip(single, (A16, At16, B16, Bt16)))
    assert torch.equal(A_cat, torch.cat([a[0].to(dtype) for a in adapters[:3]]))


def _fwd_case(M, K, N, gs, r, dtype, s=2.0, bias=False, seed=0):
    w = make_gptq(K, N, gs, seed=seed)
    x = randn((M, K), 2 + seed, dtype)
    A, B = olora.make_lora(K, N, r, 1 + seed) if r else (None, None)
    b = randn((N,), 9, dtype, 0.1) if bias else None
    return w, x, A, B, b, s


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,N,gs,r,bias", [
    (512, 2048, 2048, 128, 16, False),
    (256, 256, 256, 128, 16, True),
    (200, 1024, 1056, 64, 8, False),   # ragged M, N not a multiple of the 256-wide tile
    (128, 2048, 2048, 128, 0, False),  # adapters disabled: base only
    (300, 96, 64, 32 * 2, 32, True),   # K not a multiple of the 64-wide stage
    (64, 512, 512, 512, 64, False),    # one group (group_size == K), rank 64
])
def test_fwd_linear(M, K, N, gs, r, bias, dtype):
    import fmsa_hip

    w, x, A, B, b, s = _fwd_case(M, K, N, gs, r, dtype, bias=bias)
    ref = olora.lora_linear(x.float(), w["dense"], None if A is None else A.to(dtype).float(),
                            None if B is None else B.to(dtype).float(), s, None if b is None else b.float())
    gw = gweight(w)
    xd = dev(x)
    p = {"w": gw, "r": r, "s": s, "bias": None if b is None else dev(b)}
    if r:
        Ad, Bd = dev(A.to(dtype)), dev(B.to(dtype))
        p["U"] = fmsa_hip.lora_down(xd, Ad)
        p["B"] = Bd
    (y,) = fmsa_hip.gptq_lora_fwd(xd, [p])
    err = olora.max_rel_err(y.cpu(), ref)
    assert err < TOL, err
    if dtype == torch.float16 and gs % 64 == 0:
        # the packed-half unpack of the interleaved copy forms the same fp16 weights: identical products, bit for bit
        (y_il,) = fmsa_hip.gptq_lora_fwd(xd, [{**p, "w": gweight(w, interleaved=True)}])
        assert torch.equal(y_il, y)


def _proj_fwd(w, x_dev, A, B, s, dtype, interleaved=False):
    import fmsa_hip

    p = {"w": gweight(w, interleaved=interleaved), "r": A.shape[0], "s": s, "bias": None}
    p["U"] = fmsa_hip.lora_down(x_dev, dev(A.to(dtype)))
    p["B"] = dev(B.to(dtype))
    return p


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fwd_qkv_shared_input(dtype):
    """q 1024->1024, k/v 1024->256 (GQA-like), one launch over the concatenated N."""
    import fmsa_hip

    M, K, r, s = 384, 1024, 16, 2.0
    Ns = [1024, 256, 288]
    x = randn((M, K), 2, dtype)
    xd = dev(x)
    ws = [make_gptq(K, N, 128, seed=10 + i) for i, N in enumerate(Ns)]
    ABs = [olora.make_lora(K, N, r, 20 + i) for i, N in enumerate(Ns)]
    projs = [_proj_fwd(w, xd, A, B, s, dtype) for w, (A, B) in zip(ws, ABs)]
    outs = fmsa_hip.gptq_lora_fwd(xd, projs)
    for w, (A, B), y in zip(ws, ABs, outs):
        ref = olora.lora_linear(x.float(), w["dense"], A.to(dtype).float(), B.to(dtype).float(), s)
        assert olora.max_rel_err(y.cpu(), ref) < TOL
    if dtype == torch.float16:
        outs_il = fmsa_hip.gptq_lora_fwd(xd, [_proj_fwd(w, xd, A, B, s, dtype, True) for w, (A, B) in zip(ws, ABs)])
        assert all(torch.equal(a, b) for a, b in zip(outs_il, outs))
        # one nibble order per launch
        mixed = [_proj_fwd(w, xd, A, B, s, dtype, i == 1) for i, (w, (A, B)) in enumerate(zip(ws, ABs))]
        with pytest.raises(fmsa_hip.FmsaError):
            fmsa_hip.gptq_lora_fwd(xd, mixed)
    else:
        with pytest.raises(fmsa_hip.FmsaError):  # the interleaved copy is for fp16 activations only
            fmsa_hip.gptq_lora_fwd(xd, [_proj_fwd(w, xd, A, B, s, dtype, True) for w, (A, B) in zip(ws, ABs)])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,H,I", [(256, 512, 1024), (200, 256, 352)])
def test_fwd_swiglu(M, H, I, dtype):
    import fmsa_hip

    r, s = 16, 1.0
    x = randn((M, H), 2, dtype)
    xd = dev(x)
    wg, wu = make_gptq(H, I, 128, seed=1), make_gptq(H, I, 128, seed=2)
    (Ag, Bg), (Au, Bu) = olora.make_lora(H, I, r, 3), olora.make_lora(H, I, r, 4)
    e, g, h = fmsa_hip.gptq_lora_fwd(xd, [_proj_fwd(wg, xd, Ag, Bg, s, dtype), _proj_fwd(wu, xd, Au, Bu, s, dtype)],
                                     fmsa_hip.FWD_SWIGLU)
    e_ref = olora.lora_linear(x.float(), wg["dense"], Ag.to(dtype).float(), Bg.to(dtype).float(), s)
    g_ref = olora.lora_linear(x.float(), wu["dense"], Au.to(dtype).float(), Bu.to(dtype).float(), s)
    assert olora.max_rel_err(e.cpu(), e_ref) < TOL
    assert olora.max_rel_err(g.cpu(), g_ref) < TOL
    # h must be the reference's SwiGLU of the STORED e, g (same rounding points)
    h_ref = olora.swiglu_fwd(e.cpu(), g.cpu())
    assert olora.max_rel_err(h.cpu(), h_ref.float()) < 4e-3
    assert olora.max_rel_err(h.cpu(), torch.nn.functional.silu(e_ref) * g_ref) < TOL
    if dtype == torch.float16:
        il = fmsa_hip.gptq_lora_fwd(xd, [_proj_fwd(wg, xd, Ag, Bg, s, dtype, True), _proj_fwd(wu, xd, Au, Bu, s, dtype, True)],
                                    fmsa_hip.FWD_SWIGLU)
        assert all(torch.equal(a, b) for a, b in zip(il, (e, g, h)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("scale_mul", [1.0, 2.0 ** -12, 2.0 ** 11])
@pytest.mark.parametrize("v1", [False, True])
def test_gemm_operands_are_the_dequantised_weight_bit_for_bit(dtype, scale_mul, v1):
    """One-hot activations read the MFMA operand the kernels form straight back: with X = I the forward's output is
    deq(W), with dY = I the input gradient is deq(W)^T, each entry one exact product, so both must equal the oracle's
    dequantised weight (one rounding of the exact product to the activation type) bit for bit -- on the checkpoint
    layout, on the transposed twin, and for fp16 through the packed-half routes (interleaved copy, negzp_f16 table).
    Scales 2^-12 smaller put many products among fp16's subnormals, 2^11 larger near the top of its range."""
    import numpy as np

    import fmsa_hip

    K, N, gs = 256, 512, 64
    w = make_gptq(K, N, gs, seed=17, v1=v1)
    w["np"]["scales"] = (w["np"]["scales"].astype(np.float32) * scale_mul).astype(np.float16)
    assert np.isfinite(w["np"]["scales"]).all() and (w["np"]["scales"] != 0).all()
    w["t"]["scales"] = torch.from_numpy(w["np"]["scales"].copy())
    name = {torch.bfloat16: "bf16", torch.float16: "fp16"}[dtype]
    want = ogptq.dequant(w["np"]["qweight"], w["np"]["scales"], w["np"]["qzeros"], w["np"]["g_idx"],
                         zero_offset=w["zero_offset"], out=name)
    if dtype == torch.float16 and scale_mul < 1:
        assert (want.float().abs() < 2.0 ** -14).float().mean() > 0.2   # the case does reach the subnormals
    eye_k, eye_n = dev(torch.eye(K, dtype=dtype)), dev(torch.eye(N, dtype=dtype))
    base = {"r": 0, "s": 0.0, "bias": None}
    routes = [False] + ([True] if dtype == torch.float16 else [])
    for interleaved in routes:
        (y,) = fmsa_hip.gptq_lora_fwd(eye_k, [{**base, "w": gweight(w, interleaved=interleaved)}])
        assert torch.equal(y.cpu(), want), ("forward", interleaved)
    gw = gweight(w)
    pb = {"w": gw, "nsz": fmsa_hip.gptq_make_nsz(gw, eye_n.device), "r": 0, "s": 0.0, "dY": eye_n, "mask_src": None}
    twin = _twin(w)
    for extra in ({}, {**twin, "negzp_f16": None}, twin):
        dx = fmsa_hip.gptq_lora_bwd_dx([{**pb, **extra}], N, K)
        assert torch.equal(dx.cpu(), want.t()), ("input gradient", sorted(k for k, v in extra.items() if v is not None))


def _twin(w):
    """The weight's transposed twin for the input-gradient kernel (packed along N, fp32 scales); None, None when a
    group does not hold whole 64-column tiles (the kernel then reads the checkpoint layout)."""
    import fmsa_hip

    if w["group_size"] % 64 != 0:
        return {"qweight_t": None, "scale_f32": None, "negzp_f16": None}
    return {"qweight_t": fmsa_hip.gptq_transpose(w["dev"]["qweight"]), "scale_f32": w["dev"]["scales"].float().contiguous(),
            "negzp_f16": fmsa_hip.gptq_negzp_f16(w["dev"]["qzeros"], w["N"], w["zero_offset"])}


def _proj_bwd(w, dy_dev, A, B, s, dtype, mask_src=None, twin=False):
    import fmsa_hip

    gw = gweight(w)
    p = {"w": gw, "nsz": fmsa_hip.gptq_make_nsz(gw, dy_dev.device), "r": A.shape[0], "s": s, "dY": dy_dev,
         "mask_src": mask_src}
    if twin:
        p.update(_twin(w))
    p["T"] = fmsa_hip.lora_down(dy_dev, dev(B.to(dtype).t().contiguous()))
    p["At"] = dev(A.to(dtype).t().contiguous())
    return p


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,N,gs,r", [
    (512, 2048, 2048, 128, 16),
    (200, 1056, 1024, 64, 8),   # ragged M; K not a multiple of the 256-wide output tile
    (256, 256, 96, 128, 64),    # N not a multiple of the 64-wide stage
])
@pytest.mark.parametrize("twin", [False, True])
def test_bwd_dx_linear(M, K, N, gs, r, dtype, twin):
    import fmsa_hip

    s = 2.0
    w = make_gptq(K, N, gs, seed=3)
    A, B = olora.make_lora(K, N, r, 4)
    x = randn((M, K), 2, dtype)
    x[::7, ::5] = 0  # exact zeros: the LoRA part of dX is masked there
    dy = randn((M, N), 3, dtype)
    dyd = dev(dy)
    dx = fmsa_hip.gptq_lora_bwd_dx([_proj_bwd(w, dyd, A, B, s, dtype, mask_src=dev(x), twin=twin)], M, K)
    ref, _, _ = olora.lora_w_manual(x.float(), w["dense"], A.to(dtype).float(), B.to(dtype).float(), s, dy.float())
    assert olora.max_rel_err(dx.cpu(), ref) < TOL
    # without the mask source the LoRA term is applied everywhere
    dx2 = fmsa_hip.gptq_lora_bwd_dx([_proj_bwd(w, dyd, A, B, s, dtype, twin=twin)], M, K)
    ref2 = dy.float() @ w["dense"].t() + (dy.float() @ B.to(dtype).float()) @ (s * A.to(dtype).float())
    assert olora.max_rel_err(dx2.cpu(), ref2) < TOL


def _random_shapes(n, seed):
    """Seeded shapes that respect the kernels' contract (K, N multiples of 32; group size a multiple of 32
    dividing K; rank a multiple of 8) and otherwise hit every tail: token counts from 1, tiles cut in M, N and K."""
    import random

    rng = random.Random(seed)
    cases = []
    for _ in range(n):
        K = 32 * rng.randint(1, 40)
        gs = rng.choice([g for g in (32, 64, 96, 128, 256, K) if K % g == 0])
        cases.append((rng.choice([1, 7, 31, 64, 100, 255, 256, 257, 300, 513]), K, 32 * rng.randint(1, 40), gs,
                      rng.choice([0, 8, 16, 24, 40]), rng.random() < 0.4, rng.choice([torch.bfloat16, torch.float16])))
    return cases


@pytest.mark.parametrize("M,K,N,gs,r,bias,dtype", _random_shapes(20, 1234))
def test_fwd_and_bwd_random_shapes(M, K, N, gs, r, bias, dtype):
    import fmsa_hip

    s = 0.5
    w = make_gptq(K, N, gs, seed=K + N)
    gw = gweight(w)
    x = randn((M, K), 2, dtype)
    x[::3, ::4] = 0
    A, B = olora.make_lora(K, N, r, 5) if r else (None, None)
    Aq, Bq = (A.to(dtype).float(), B.to(dtype).float()) if r else (None, None)
    b = randn((N,), 9, dtype, 0.1) if bias else None
    xd = dev(x)
    p = {"w": gw, "r": r, "s": s, "bias": None if b is None else dev(b)}
    if r:
        p["U"] = fmsa_hip.lora_down(xd, dev(A.to(dtype)))
        p["B"] = dev(B.to(dtype))
    (y,) = fmsa_hip.gptq_lora_fwd(xd, [p])
    ref = olora.lora_linear(x.float(), w["dense"], Aq, Bq, s, None if b is None else b.float())
    assert olora.max_rel_err(y.cpu(), ref) < TOL
    if dtype == torch.float16 and gs % 64 == 0:  # the packed-half unpack of the interleaved copy: the same bits
        (y_il,) = fmsa_hip.gptq_lora_fwd(xd, [{**p, "w": gweight(w, interleaved=True)}])
        assert torch.equal(y_il, y)
    dy = randn((M, N), 3, dtype)
    dyd = dev(dy)
    if r:
        dx = fmsa_hip.gptq_lora_bwd_dx([_proj_bwd(w, dyd, A, B, s, dtype, mask_src=xd)], M, K)
        # the kernel flavour that reads the transposed twin: same values in the same order, so the same bits
        dx_t = fmsa_hip.gptq_lora_bwd_dx([_proj_bwd(w, dyd, A, B, s, dtype, mask_src=xd, twin=True)], M, K)
        assert torch.equal(dx, dx_t)
        dx_ref, dA_ref, dB_ref = olora.lora_w_manual(x.float(), w["dense"], Aq, Bq, s, dy.float())
        T = fmsa_hip.lora_down(dyd, dev(B.to(dtype).t().contiguous()))
        dA, dB = fmsa_hip.lora_grad_batch([(T, xd, s, False, torch.float32), (p["U"], dyd, s, True, torch.float32)])
        assert olora.max_rel_err(dA.cpu(), dA_ref) < TOL and olora.max_rel_err(dB.cpu(), dB_ref) < TOL
    else:
        base = {"w": gw, "nsz": fmsa_hip.gptq_make_nsz(gw, dyd.device), "dY": dyd, "T": None, "At": None,
                "mask_src": None, "r": 0, "s": 0.0}
        dx = fmsa_hip.gptq_lora_bwd_dx([base], M, K)
        assert torch.equal(dx, fmsa_hip.gptq_lora_bwd_dx([{**base, **_twin(w)}], M, K))
        dx_ref = dy.float() @ w["dense"].t()
    assert olora.max_rel_err(dx.cpu(), dx_ref) < TOL


@pytest.mark.parametrize("dtype", [torch.bfloat16])
def test_bwd_dx_three_projections(dtype):
    import fmsa_hip

    M, K, r, s = 320, 1024, 16, 2.0
    Ns = [1024, 256, 288]
    x = randn((M, K), 2, dtype)
    x[::5, ::3] = 0  # masked entries: no LoRA contribution from any projection
    ws = [make_gptq(K, N, 128, seed=10 + i) for i, N in enumerate(Ns)]
    ABs = [olora.make_lora(K, N, r, 20 + i) for i, N in enumerate(Ns)]
    dys = [randn((M, N), 30 + i, dtype) for i, N in enumerate(Ns)]
    xd = dev(x)  # one mask source for the whole call
    projs = [_proj_bwd(w, dev(dy), A, B, s, dtype, mask_src=xd) for w, (A, B), dy in zip(ws, ABs, dys)]
    dx = fmsa_hip.gptq_lora_bwd_dx(projs, M, K)
    twins = [_proj_bwd(w, dev(dy), A, B, s, dtype, mask_src=xd, twin=True) for w, (A, B), dy in zip(ws, ABs, dys)]
    assert torch.equal(dx, fmsa_hip.gptq_lora_bwd_dx(twins, M, K))
    # a call in which one projection comes without its twin takes the checkpoint-layout kernel for all of them
    assert torch.equal(dx, fmsa_hip.gptq_lora_bwd_dx([twins[0], projs[1], twins[2]], M, K))
    ref, _ = olora.lora_qkv_manual(x.float(), [(w["dense"], A.to(dtype).float(), B.to(dtype).float(), s)
                                                 for w, (A, B) in zip(ws, ABs)], [d.float() for d in dys])
    assert olora.max_rel_err(dx.cpu(), ref) < TOL


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,H,I", [(256, 512, 1024), (200, 256, 352), (300, 288, 640)])
@pytest.mark.parametrize("twin", [False, True])
def test_bwd_swiglu(M, H, I, dtype, twin):
    """Down-projection backward: dh = dY Wd^T + LoRA, then the in-place SwiGLU backward."""
    import fmsa_hip

    r, s = 16, 1.0
    wd = make_gptq(I, H, 128 if I % 128 == 0 else 32 * 11, seed=5)  # down: I -> H, so K = I, N = H
    Ad, Bd = olora.make_lora(I, H, r, 6)
    e = randn((M, I), 7, dtype)
    e[::9, ::4] = 0  # h = silu(0) * g = 0 there: the LoRA part of dh is masked
    g = randn((M, I), 8, dtype)
    dy = randn((M, H), 9, dtype)
    e_d, g_d = dev(e).clone(), dev(g).clone()
    h = fmsa_hip.gptq_lora_bwd_dx([_proj_bwd(wd, dev(dy), Ad, Bd, s, dtype, twin=twin)], M, I, fmsa_hip.BWD_SWIGLU, e=e_d, g=g_d)
    h_mask = (olora.swiglu_fwd(e, g) != 0).float()
    dh_ref = dy.float() @ wd["dense"].t() + h_mask * ((dy.float() @ Bd.to(dtype).float()) @ (s * Ad.to(dtype).float()))
    # h does not depend on the GEMM: it must match the reference's rounding points closely
    h_ref, _, _ = olora.swiglu_bwd(dh_ref.to(dtype), e, g)
    assert olora.max_rel_err(h.cpu(), h_ref.float()) < 4e-3
    # d_g, d_e against the un-rounded fp32 math (the kernel rounds dh, dh*g and the results to the
    # storage type as the reference does; each rounding is <= 2^-9 relative)
    e32, g32 = e.float(), g.float()
    se = torch.sigmoid(e32)
    dg_ref = dh_ref * (se * e32)
    de_ref = dh_ref * g32 * se * (1.0 + e32 * (1.0 - se))
    assert olora.max_rel_err(e_d.cpu(), dg_ref) < TOL
    assert olora.max_rel_err(g_d.cpu(), de_ref) < TOL


@pytest.mark.parametrize("K,N", [(32, 32), (256, 96), (1056, 1024)])
def test_gptq_interleave_bit_exact(K, N):
    """Word [k8, n] of the interleaved copy holds q[8 k8 + e, n], element 2p at nibble position p and 2p + 1 at 4 + p."""
    import numpy as np

    import fmsa_hip

    w = make_gptq(K, N, 32, seed=K + 5 * N)
    q = ogptq.unpack_rows(w["np"]["qweight"]).astype(np.uint32)  # [K, N]
    want = np.zeros((K // 8, N), dtype=np.uint32)
    for j in range(8):
        want |= q[j::8, :] << np.uint32(4 * (j // 2 + 4 * (j % 2)))
    got = fmsa_hip.gptq_interleave(dev(w["t"]["qweight"])).cpu().numpy().view(np.uint32)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("K,N", [(32, 32), (256, 96), (1056, 1024)])
def test_gptq_transpose_bit_exact(K, N):
    """The twin's packing: word [n8, k] holds q[k, 8 n8 + e], element 2p at nibble position p and 2p + 1 at 4 + p,
    against a plain numpy re-packing of the unpacked 4-bit values (the unpack is the oracle's, which the layout tests
    pin bit by bit)."""
    import numpy as np

    import fmsa_hip

    w = make_gptq(K, N, 32, seed=K + 3 * N)
    q = ogptq.unpack_rows(w["np"]["qweight"]).astype(np.uint32)  # [K, N]
    want = np.zeros((N // 8, K), dtype=np.uint32)
    for j in range(8):  # element j of a word: even elements fill the low half-word, odd ones the high half
        want |= q[:, j::8].T << np.uint32(4 * (j // 2 + 4 * (j % 2)))
    got = fmsa_hip.gptq_transpose(dev(w["t"]["qweight"])).cpu().numpy().view(np.uint32)
    assert np.array_equal(got, want)
