"""GPU parity of the 256x128 GEMM kernel for two workgroups per CU (tileConfig bit 11) against the oracle (int8, bit-exact) and against
the 256x256 ring kernel, whose own parity tests are in test_gemm_gpu.py: the two kernels add the same products in the same order per
accumulator, so every result type must agree bit for bit."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from oracle_lib import Oracle, _ptr  # noqa: E402

TWIN = 2048


@pytest.fixture(scope="module")
def lib():
    import tscale2_amd
    return tscale2_amd.load()


@pytest.fixture(scope="module")
def orc():
    return Oracle()


def _e4m3(shape, g, scale=6.0):
    return (torch.randn(shape, device="cuda", generator=g) * scale).to(torch.float8_e4m3fn).view(torch.uint8)


# k = 64 .. 320 walk through every remainder of the three-stage rotation (k / 64 = 1, 2, 3, 4, 5 steps)
@pytest.mark.parametrize("m,n,k", [(256, 128, 64), (256, 128, 128), (512, 384, 192), (256, 256, 256), (768, 128, 320), (512, 640, 1024),
                                   (256, 128, 4096)])
def test_int8_int32_sums_are_exact(lib, orc, m, n, k):
    print(f"case twin int8 exact m={m} n={n} k={k}", flush=True)
    from tscale2_amd import lib as L
    r = np.random.default_rng(m + n + k)
    a = r.integers(-128, 128, (m, k), dtype=np.int8)
    b = r.integers(-128, 128, (n, k), dtype=np.int8)
    ref = np.empty((m, n), np.int32)
    orc.lib.orc_gemm_i8_nt(_ptr(a), _ptr(b), _ptr(ref), m, n, k)
    tc = torch.full((m, n), -7, dtype=torch.int32, device="cuda")
    lib.gemm_nt(torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), tc, L.I8, L.I32, tile_config=TWIN)
    torch.cuda.synchronize()
    assert np.array_equal(tc.cpu().numpy(), ref)


def test_int8_row_scaled_results_equal_the_ring_kernel(lib):
    print("case twin int8 rowscale", flush=True)
    from tscale2_amd import lib as L
    m, n, k = 512, 256, 448
    g = torch.Generator(device="cuda").manual_seed(3)
    a = torch.randint(-127, 128, (m, k), dtype=torch.int8, device="cuda", generator=g)
    b = torch.randint(-127, 128, (n, k), dtype=torch.int8, device="cuda", generator=g)
    rs = torch.rand(m, device="cuda", generator=g) + 0.1
    c0 = torch.randn((m, n), device="cuda", generator=g)
    for epi, m_live in ((L.EPI_STORE, 0), (L.EPI_STORE, 300), (L.EPI_ADD, 0), (L.EPI_ADD, 300)):
        want, got = c0.clone(), c0.clone()
        # (k = 448 is not a multiple of 128: the reference kernel here is the 128x128 two-stage loop on k = 384 + a separate check below)
        lib.gemm_nt(a[:, :384].contiguous(), b[:, :384].contiguous(), want, L.I8, L.F32, row_scale=rs, alpha=0.01, epilogue=epi, tile_config=1,
                    m_live=m_live)
        lib.gemm_nt(a[:, :384].contiguous(), b[:, :384].contiguous(), got, L.I8, L.F32, row_scale=rs, alpha=0.01, epilogue=epi, tile_config=TWIN,
                    m_live=m_live)
        torch.cuda.synchronize()
        assert torch.equal(got, want), (epi, m_live)
    # a contraction of seven 64-byte steps against the int64 product
    got = torch.empty((m, n), device="cuda")
    lib.gemm_nt(a, b, got, L.I8, L.F32, row_scale=rs, alpha=0.01, tile_config=TWIN)
    torch.cuda.synchronize()
    ref = (a.cpu().numpy().astype(np.int64) @ b.cpu().numpy().astype(np.int64).T).astype(np.float64) * rs.cpu().numpy().astype(np.float64)[:, None] * 0.01
    np.testing.assert_allclose(got.cpu().numpy(), ref, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("ab", ["e4m3", "bf16"])
@pytest.mark.parametrize("m,n,k", [(256, 128, 128), (512, 384, 640), (1024, 256, 2048)])
def test_float_results_equal_the_ring_kernel_bit_for_bit(lib, ab, m, n, k):
    """fp32 store and accumulate, bf16 store and accumulate, IEEE half store; live rows short of m."""
    print(f"case twin float {ab} m={m} n={n} k={k}", flush=True)
    from tscale2_amd import lib as L
    g = torch.Generator(device="cuda").manual_seed(m + k)
    if ab == "e4m3":
        a, b, t = _e4m3((m, k), g), _e4m3((n, k), g), L.E4M3
    else:
        a = torch.randn((m, k), device="cuda", generator=g).bfloat16().view(torch.int16)
        b = torch.randn((n, k), device="cuda", generator=g).bfloat16().view(torch.int16)
        t = L.BF16
    aptr = torch.full((1,), 0.61, device="cuda")
    c0 = torch.randn((m, n), device="cuda", generator=g)
    ref_cfg = 1 if (m % 256 == 0 and n % 256 == 0) else 2
    for c_type, epi, m_live in ((L.F32, L.EPI_STORE, 0), (L.F32, L.EPI_STORE, m - 37), (L.F32, L.EPI_ADD, m - 37), (L.BF16, L.EPI_STORE, 0),
                                (L.BF16, L.EPI_STORE, m - 37), (L.BF16, L.EPI_ADD, 0), (L.F16, L.EPI_STORE, m - 5)):
        if c_type == L.F32:
            want, got = c0.clone(), c0.clone()
            wv, gv = want, got
        else:
            dt = torch.bfloat16 if c_type == L.BF16 else torch.float16
            want, got = c0.to(dt), c0.to(dt)
            wv, gv = want.view(torch.int16), got.view(torch.int16)
        lib.gemm_nt(a, b, wv, t, c_type, alpha=0.02, alpha_ptr=aptr, epilogue=epi, tile_config=ref_cfg, m_live=m_live)
        lib.gemm_nt(a, b, gv, t, c_type, alpha=0.02, alpha_ptr=aptr, epilogue=epi, tile_config=TWIN, m_live=m_live)
        torch.cuda.synchronize()
        assert torch.equal(gv, wv), (c_type, epi, m_live)
    # and the fp32 result against the fp64 product
    got = torch.empty((m, n), device="cuda")
    lib.gemm_nt(a, b, got, t, L.F32, tile_config=TWIN)
    torch.cuda.synchronize()
    if ab == "e4m3":
        fa, fb = a.view(torch.float8_e4m3fn).double(), b.view(torch.float8_e4m3fn).double()
    else:
        fa, fb = a.view(torch.bfloat16).double(), b.view(torch.bfloat16).double()
    ref = fa @ fb.T
    assert (got.double() - ref).abs().max().item() <= 1e-4 * ref.abs().max().item()


@pytest.mark.parametrize("ab", ["i8", "e4m3"])
@pytest.mark.parametrize("normalize,use_rope", [(True, True), (True, False), (False, True)])
def test_row_tile_normalize_rope_epilogue_equals_the_ring_kernel(lib, ab, normalize, use_rope):
    print("case twin norm/rope epilogue", ab, normalize, use_rope, flush=True)
    from tscale2_amd import lib as L
    m, n, k = 512, 768, 320
    g = torch.Generator(device="cuda").manual_seed(5)
    if ab == "i8":
        a = torch.randint(-90, 90, (m, k), dtype=torch.int8, device="cuda", generator=g)
        b = torch.randint(-90, 90, (n, k), dtype=torch.int8, device="cuda", generator=g)
        t = L.I8
    else:
        a, b, t = _e4m3((m, k), g, 8.0), _e4m3((n, k), g, 8.0), L.E4M3
    a[300:310] = 0
    m_live = 500
    rope = None
    if use_rope:
        ang = torch.rand((m, 64), device="cuda", generator=g) * 6.28
        rope = torch.stack([torch.cos(ang), torch.sin(ang)], dim=2).reshape(m, 128).contiguous()
    res = []
    # (k = 320: the ring kernel takes 128-byte steps, so it is given the first 256 bytes and the twin kernel both lengths)
    for cfg, kk in ((1, 256), (TWIN, 256), (TWIN, 320)):
        got = torch.full((m, n), 9, dtype=torch.int16, device="cuda")
        got_sc = torch.full((n // 128, m), -2.0, device="cuda")
        lib.gemm_nt(a[:, :kk].contiguous(), b[:, :kk].contiguous(), got, t, L.BF16, alpha=0.37, m_live=m_live, tile_config=cfg,
                    epilogue=L.EPI_ROW_TILE_NORM, normalize=normalize, vec_scale=1 / 24.0, rope=rope, tile_scale=got_sc if normalize else None)
        torch.cuda.synchronize()
        res.append((got, got_sc))
    assert torch.equal(res[0][0], res[1][0])
    if normalize:
        assert torch.equal(res[0][1][:, :m_live], res[1][1][:, :m_live])
    # the longer contraction against the two-pass path (fp32 product, then ts2_row_tile_normalize_rope): one bf16 ulp
    raw = torch.empty((m, n), dtype=torch.float32, device="cuda")
    lib.gemm_nt(a, b, raw, t, L.F32, alpha=0.37, m_live=m_live, tile_config=TWIN)
    want = torch.full((m, n), 7, dtype=torch.int16, device="cuda")
    want_sc = torch.full((n // 128, m), -1.0, device="cuda")
    L.call("ts2_row_tile_normalize_rope", m_live, m, raw, L.F32, 1.0, int(normalize), 1 / 24.0, rope, want, want_sc if normalize else None)
    wf, gf = want.view(torch.bfloat16).float(), res[2][0].view(torch.bfloat16).float()
    tile_max = wf.abs().view(m, n // 128, 128).amax(2, keepdim=True).expand(m, n // 128, 128).reshape(m, n)
    assert ((gf - wf).abs() <= wf.abs() * 2.0 ** -7 + tile_max * 2.0 ** -21 + 1e-30).all()
    assert (gf[m_live:] == 0).all() and (gf[300:310] == 0).all()


@pytest.mark.parametrize("ab,add,c_type", [("e4m3", False, "f32"), ("e4m3", True, "f32"), ("bf16", True, "f32"), ("e4m3", False, "bf16")])
def test_several_products_into_one_result_equal_the_ring_kernel(lib, ab, add, c_type):
    print("case twin several products", ab, add, c_type, flush=True)
    from tscale2_amd import lib as L
    m, n, k, nseg = 512, 768, 384, 4
    g = torch.Generator(device="cuda").manual_seed(11)
    As, Bs, alphas, ptrs = [], [], [], []
    for i in range(nseg):
        if ab == "e4m3":
            a, b, t = _e4m3((m, k), g), _e4m3((n, k), g), L.E4M3
        else:
            a = torch.randn((m, k), device="cuda", generator=g).bfloat16().view(torch.int16)
            b = torch.randn((n, k), device="cuda", generator=g).bfloat16().view(torch.int16)
            t = L.BF16
        As.append(a); Bs.append(b)
        alphas.append(0.25 * (i + 1))
        ptrs.append(None if i == 2 else torch.full((1,), 0.0 if i == 1 else 0.5 + 0.37 * i, device="cuda"))  # product 1 has a zero factor
    c0 = torch.randn((m, n), device="cuda", generator=g)
    out = []
    for cfg in (1, TWIN):
        if c_type == "f32":
            c = c0.clone(); cv = c; ct = L.F32
        else:
            c = c0.bfloat16(); cv = c.view(torch.int16); ct = L.BF16
        lib.gemm_nt(As[0], Bs[0], cv, t, ct, alpha=alphas[0], alpha_ptr=ptrs[0], epilogue=L.EPI_ADD if add else L.EPI_STORE, m_live=500,
                    tile_config=cfg, segments=[(As[i], Bs[i], alphas[i], ptrs[i]) for i in range(1, nseg)])
        torch.cuda.synchronize()
        out.append(cv)
    assert torch.equal(out[0], out[1])


def test_calls_the_kernel_cannot_run_are_refused(lib):
    from tscale2_amd import lib as L
    a = torch.zeros((384, 256), dtype=torch.int8, device="cuda")
    b = torch.zeros((128, 256), dtype=torch.int8, device="cuda")
    c = torch.zeros((384, 128), device="cuda")
    assert lib.gemm_nt(a, b, c, L.I8, L.F32, tile_config=TWIN, check=False) == -3        # m not a multiple of 256
    a = torch.zeros((256, 256), dtype=torch.int8, device="cuda")
    c = torch.zeros((256, 128), device="cuda")
    assert lib.gemm_nt(a, b, c, L.I8, L.F32, tile_config=TWIN, split_k=2, check=False) == -3
    sc = torch.zeros((1, 256), device="cuda")
    c8 = torch.zeros((256, 128), dtype=torch.int8, device="cuda")
    assert lib.gemm_nt(a, b, c8, L.I8, L.I8, tile_config=TWIN, epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=sc, check=False) == -3
