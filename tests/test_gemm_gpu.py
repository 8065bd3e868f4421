"""GPU parity of ts2_gemm_nt against the CPU oracle (bit-exact for int8, stated tolerance for fp8/bf16)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from oracle_lib import Oracle, _ptr  # noqa: E402


@pytest.fixture(scope="module")
def lib():
    import tscale2_amd
    return tscale2_amd.load()


@pytest.fixture(scope="module")
def orc():
    return Oracle()


def orc_gemm_i8(orc, a, b):
    m, k = a.shape
    n = b.shape[0]
    c = np.empty((m, n), np.int32)
    orc.lib.orc_gemm_i8_nt(_ptr(a), _ptr(b), _ptr(c), m, n, k)
    return c


@pytest.mark.parametrize("m,n,k,cfg", [(128, 128, 128, 0), (256, 384, 512, 2), (512, 256, 1024, 1), (1024, 768, 256, 0), (256, 256, 4096, 1)])
def test_int8_int32_bit_exact(lib, orc, m, n, k, cfg):
    print(f"case int8 exact m={m} n={n} k={k} cfg={cfg}", flush=True)
    r = np.random.default_rng(m + n + k)
    a = r.integers(-128, 128, (m, k), dtype=np.int8)
    b = r.integers(-128, 128, (n, k), dtype=np.int8)
    ref = orc_gemm_i8(orc, a, b)
    from tscale2_amd import lib as L
    ta, tb = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    tc = torch.full((m, n), -7, dtype=torch.int32, device="cuda")
    lib.gemm_nt(ta, tb, tc, L.I8, L.I32, tile_config=cfg)
    torch.cuda.synchronize()
    assert np.array_equal(tc.cpu().numpy(), ref)


@pytest.mark.parametrize("cfg", [1, 2])
def test_int8_rowscale_store_and_add(lib, orc, cfg):
    print(f"case int8 rowscale cfg={cfg}", flush=True)
    from tscale2_amd import lib as L
    m, n, k = 512, 256, 384 if cfg == 2 else 512
    r = np.random.default_rng(5)
    a = r.integers(-127, 128, (m, k), dtype=np.int8)
    b = r.integers(-127, 128, (n, k), dtype=np.int8)
    rs = r.random(m).astype(np.float32) + 0.1
    c0 = r.standard_normal((m, n)).astype(np.float32)
    alpha = 0.01
    ref = c0.copy()
    orc.lib.orc_gemm_i8_nt_rowscale(_ptr(a), _ptr(rs), _ptr(b), C.c_float(alpha), _ptr(ref), m, n, k, 1)
    ta, tb, trs = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(rs).cuda()
    tc = torch.from_numpy(c0).cuda()
    lib.gemm_nt(ta, tb, tc, L.I8, L.F32, row_scale=trs, alpha=alpha, epilogue=L.EPI_ADD, tile_config=cfg)
    torch.cuda.synchronize()
    # the int32 sum is exact; the fp32 epilogue multiplies in a different order than the oracle: <= 2 ulp of the product
    np.testing.assert_allclose(tc.cpu().numpy(), ref, rtol=3e-7 * 4, atol=1e-6)
    tc2 = torch.empty_like(tc)
    lib.gemm_nt(ta, tb, tc2, L.I8, L.F32, row_scale=trs, alpha=alpha, epilogue=L.EPI_STORE, tile_config=cfg, m_live=300)
    torch.cuda.synchronize()
    got = tc2.cpu().numpy()
    np.testing.assert_allclose(got[:300], (ref - c0)[:300], rtol=1e-5, atol=2e-6)
    assert np.all(got[300:] == 0)


def test_int8_ktile_scale(lib, orc):
    print("case int8 ktile", flush=True)
    from tscale2_amd import lib as L
    m, n, k, kt = 256, 128, 1024, 256
    r = np.random.default_rng(6)
    a = r.integers(-127, 128, (m, k), dtype=np.int8)
    b = r.integers(-127, 128, (n, k), dtype=np.int8)
    ks = (r.random(k // kt).astype(np.float32) + 0.5) * 1e-3
    ref = np.empty((m, n), np.float32)
    orc.lib.orc_gemm_i8_nt_ktile(_ptr(a), _ptr(b), _ptr(ks), kt, C.c_float(0.5), _ptr(ref), m, n, k)
    ta, tb, tks = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(ks).cuda()
    tc = torch.empty((m, n), dtype=torch.float32, device="cuda")
    lib.gemm_nt(ta, tb, tc, L.I8, L.F32, k_tile_scale=tks, k_tile=kt, alpha=0.5)
    torch.cuda.synchronize()
    # tiles are added in the same order in fp32; fma contraction on the device may differ by an ulp per tile
    np.testing.assert_allclose(tc.cpu().numpy(), ref, rtol=2e-6, atol=1e-4)


def test_fp8_and_bf16_against_fp64(lib, orc):
    print("case fp8/bf16", flush=True)
    from tscale2_amd import lib as L
    m, n, k = 256, 256, 512
    r = np.random.default_rng(7)
    tab = Oracle().e4m3_table()
    codes_a = r.integers(0, 256, (m, k)).astype(np.uint8)
    codes_b = r.integers(0, 256, (n, k)).astype(np.uint8)
    codes_a[(codes_a & 0x7f) == 0x7f] = 0  # NaN codes of OCP e4m3
    codes_b[(codes_b & 0x7f) == 0x7f] = 0
    fa, fb = tab[codes_a].astype(np.float64), tab[codes_b].astype(np.float64)
    ref = fa @ fb.T
    for cfg in (1, 2):
        tc = torch.empty((m, n), dtype=torch.float32, device="cuda")
        lib.gemm_nt(torch.from_numpy(codes_a).cuda(), torch.from_numpy(codes_b).cuda(), tc, L.E4M3, L.F32, tile_config=cfg)
        torch.cuda.synchronize()
        # uniformly random codes span 2^-9..448: the worst case for the MFMA fp8 adder tree, which aligns the 64 products of one
        # instruction to their largest exponent before adding.  Measured 7e-5 of max|C| here; bound stated at 2e-4 (the north-star
        # tolerance for fp8 outputs is 1e-2).  Gaussian operands are checked at 1e-4 below.
        assert np.abs(tc.cpu().numpy() - ref).max() <= 2e-4 * np.abs(ref).max()
        ga = np.array([orc.lib.orc_cvt_e4m3_rne(C.c_float(v)) for v in (r.standard_normal(m * k) * 8)], np.uint8).reshape(m, k)
        gb = np.array([orc.lib.orc_cvt_e4m3_rne(C.c_float(v)) for v in (r.standard_normal(n * k) * 8)], np.uint8).reshape(n, k)
        ref_g = tab[ga].astype(np.float64) @ tab[gb].astype(np.float64).T
        lib.gemm_nt(torch.from_numpy(ga).cuda(), torch.from_numpy(gb).cuda(), tc, L.E4M3, L.F32, tile_config=cfg)
        torch.cuda.synchronize()
        assert np.abs(tc.cpu().numpy() - ref_g).max() <= 1e-4 * np.abs(ref_g).max()  # measured 4e-5
    # bf16
    k2 = 256
    xa = torch.from_numpy(r.standard_normal((m, k2)).astype(np.float32)).cuda().bfloat16()
    xb = torch.from_numpy(r.standard_normal((n, k2)).astype(np.float32)).cuda().bfloat16()
    ref2 = xa.double().cpu().numpy() @ xb.double().cpu().numpy().T
    for cfg in (1, 2):
        tc = torch.empty((m, n), dtype=torch.float32, device="cuda")
        lib.gemm_nt(xa.view(torch.int16), xb.view(torch.int16), tc, L.BF16, L.F32, tile_config=cfg)
        torch.cuda.synchronize()
        assert np.abs(tc.cpu().numpy() - ref2).max() <= 1e-5 * np.abs(ref2).max() + 1e-4
        tb16 = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        lib.gemm_nt(xa.view(torch.int16), xb.view(torch.int16), tb16.view(torch.int16), L.BF16, L.BF16, tile_config=cfg, alpha=0.5)
        torch.cuda.synchronize()
        # bf16 output: relative error <= 2^-8 of each value
        np.testing.assert_allclose(tb16.float().cpu().numpy(), 0.5 * ref2, rtol=2 ** -8, atol=1e-3)


def test_packed_delta_epilogue(lib, orc):
    print("case packed delta", flush=True)
    from tscale2_amd import lib as L
    for cfg, (m, n, k) in ((1, (256, 256, 256)), (2, (128, 256, 256))):
        r = np.random.default_rng(8 + cfg)
        a = r.integers(-127, 128, (m, k), dtype=np.int8)
        b = r.integers(-127, 128, (n, k), dtype=np.int8)
        a[5] = 0  # a zero row -> zero tiles
        acc = orc_gemm_i8(orc, a, b).astype(np.float32) * np.float32(0.25)
        delta = np.zeros((m, n), np.int8)
        ts = np.zeros((n // 128, m), np.float32)
        orc.lib.orc_compress_delta(_ptr(acc), _ptr(delta), _ptr(ts), m, n)
        tc = torch.zeros((m, n), dtype=torch.int8, device="cuda")
        tts = torch.full((n // 128, m), -1.0, dtype=torch.float32, device="cuda")
        lib.gemm_nt(torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), tc, L.I8, L.I8, alpha=0.25,
                    epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=tts, tile_config=cfg)
        torch.cuda.synchronize()
        np.testing.assert_allclose(tts.cpu().numpy(), ts, rtol=2e-7)
        # bytes: identical except where v/scale lands within an ulp of a rounding boundary
        diff = np.abs(tc.cpu().numpy().astype(np.int32) - delta)
        assert diff.max() <= 1 and (diff != 0).mean() < 1e-3


@pytest.mark.parametrize("k_major", [False, True])
def test_packed_delta_epilogue_equals_the_packed_fp32_product(lib, k_major):
    """e4m3 operands on the 256x256 tile: the fused ROW_TILE_MAXNORM epilogue against the same product stored in fp32 and packed by
    ts2_pack_delta (the same arithmetic on the same fp32 sums: bit-identical bytes and scales), with a scale behind a pointer; live
    rows short of m (bytes and scales of the rest are zero); and results whose rows start off the 16-byte and off the 4-byte grid
    (the epilogue stores 16 bytes per lane where it can), nothing written past a row's end."""
    print("case packed delta against pack_delta", k_major, flush=True)
    import ctypes as C
    from tscale2_amd import lib as L
    m, n, k = 512, 768, 640
    g = torch.Generator(device="cuda").manual_seed(77)

    def codes(shape):
        return (torch.randint(0, 120, shape, device="cuda", generator=g) | (torch.randint(0, 2, shape, device="cuda", generator=g) << 7)).to(torch.uint8)
    a, b = (codes((k, m)), codes((k, n))) if k_major else (codes((m, k)), codes((n, k)))
    if k_major:
        a[:, 7] = 0
    else:
        a[7] = 0                                                    # a zero row: zero tiles, zero scales
    kw = dict(m=m, n=n, k=k, k_major=True) if k_major else {}
    sc = torch.tensor([1.7], device="cuda")
    raw = torch.zeros((m, n), device="cuda")
    lib.gemm_nt(a, b, raw, L.E4M3, L.F32, tile_config=1, **kw)
    want = torch.zeros((m, n), dtype=torch.int8, device="cuda"); want_ts = torch.zeros((n // 128, m), device="cuda")
    L.call("ts2_pack_delta", raw, 1, C.c_int64(0), m, n, 0.03, sc, want, want_ts)
    got = torch.full((m, n), 3, dtype=torch.int8, device="cuda"); got_ts = torch.full((n // 128, m), -1.0, device="cuda")
    lib.gemm_nt(a, b, got, L.E4M3, L.I8, alpha=0.03, alpha_ptr=sc, epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=got_ts, tile_config=1, **kw)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and torch.equal(got_ts, want_ts)
    assert int(got.abs().max()) == 127 and bool((got[7] == 0).all()) and bool((got_ts[:, 7] == 0).all())
    for pad in (4, 1):                                              # row stride n + pad bytes
        wide = torch.full((m, n + pad), 5, dtype=torch.int8, device="cuda")
        ts2 = torch.full((n // 128, m), -1.0, device="cuda")
        lib.gemm_nt(a, b, wide[:, :n], L.E4M3, L.I8, alpha=0.03, alpha_ptr=sc, epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=ts2, tile_config=1, **kw)
        torch.cuda.synchronize()
        assert torch.equal(wide[:, :n], want) and torch.equal(ts2, want_ts) and bool((wide[:, n:] == 5).all())
    if not k_major:
        live = 300
        lib.gemm_nt(a, b, got, L.E4M3, L.I8, alpha=0.03, alpha_ptr=sc, epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=got_ts, tile_config=1, m_live=live)
        torch.cuda.synchronize()
        assert torch.equal(got[:live], want[:live]) and torch.equal(got_ts[:, :live], want_ts[:, :live])
        assert bool((got[live:] == 0).all()) and bool((got_ts[:, live:] == 0).all())


def test_split_k_matches(lib, orc):
    print("case split-k", flush=True)
    from tscale2_amd import lib as L
    m, n, k = 256, 256, 2048
    r = np.random.default_rng(9)
    a = r.integers(-16, 17, (m, k), dtype=np.int8)
    b = r.integers(-16, 17, (n, k), dtype=np.int8)
    ref = orc_gemm_i8(orc, a, b).astype(np.float32)  # |sum| < 2^24: every fp32 partial sum is exact
    ta, tb = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    tc = torch.full((4 * m, n), 3.0, dtype=torch.float32, device="cuda")
    lib.gemm_nt(ta, tb, tc, L.I8, L.F32, split_k=4, split_slab_bytes=m * n * 4, m=m, n=n, k=k)
    torch.cuda.synchronize()
    slices = tc.cpu().numpy().reshape(4, m, n)
    for i in range(4):  # every stored slice is the product over its quarter of the contraction
        assert np.array_equal(slices[i], orc_gemm_i8(orc, np.ascontiguousarray(a[:, i * 512:(i + 1) * 512]), np.ascontiguousarray(b[:, i * 512:(i + 1) * 512])).astype(np.float32)), i
    assert np.array_equal(slices.sum(0), ref)
    # slices are stored, never added atomically: without a slab the call is refused
    assert lib.gemm_nt(ta, tb, tc[:m], L.I8, L.F32, split_k=4, check=False) == -3


def test_rejects_bad_shapes(lib):
    from tscale2_amd import lib as L
    a = torch.zeros((128, 100), dtype=torch.int8, device="cuda")
    c = torch.zeros((128, 128), dtype=torch.float32, device="cuda")
    assert lib.gemm_nt(a, a, c, L.I8, L.F32, check=False) == -1
    a2 = torch.zeros((100, 128), dtype=torch.int8, device="cuda")
    assert lib.gemm_nt(a2, a2, c, L.I8, L.F32, check=False) == -1


def test_eight_wave_configuration_is_bit_exact(lib, orc):
    print("case 8-wave config", flush=True)
    from tscale2_amd import lib as L
    m, n, k = 512, 256, 768
    r = np.random.default_rng(10)
    a = r.integers(-128, 128, (m, k), dtype=np.int8)
    b = r.integers(-128, 128, (n, k), dtype=np.int8)
    ref = orc_gemm_i8(orc, a, b).astype(np.float32)  # fp32 store of exact int32 sums (|sum| < 2^24 here)
    tc = torch.empty((m, n), dtype=torch.float32, device="cuda")
    lib.gemm_nt(torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), tc, L.I8, L.F32, tile_config=9)
    torch.cuda.synchronize()
    assert np.array_equal(tc.cpu().numpy(), ref.astype(np.float32))


@pytest.mark.parametrize("ab", ["i8", "e4m3"])
@pytest.mark.parametrize("normalize,use_rope", [(True, True), (True, False), (False, True)])
def test_fused_row_tile_normalize_rope_epilogue_matches_the_two_pass_path(ab, normalize, use_rope):
    """TS2_EPI_ROW_TILE_NORM against the same product stored in fp32 followed by ts2_row_tile_normalize_rope: same arithmetic except
    for the order of the 128 squares in the tile sum, so the bf16 results differ by one unit in the last place at most (or by fp32
    rounding of the tile's largest values where the rotation cancels)."""
    print("case fused norm/rope epilogue", ab, normalize, use_rope, flush=True)
    from tscale2_amd import lib as L
    lib = L.load()
    m, n, k = 512, 768, 256
    g = torch.Generator(device="cuda").manual_seed(5)
    if ab == "i8":
        a = torch.randint(-90, 90, (m, k), dtype=torch.int8, device="cuda", generator=g)
        b = torch.randint(-90, 90, (n, k), dtype=torch.int8, device="cuda", generator=g)
        t = L.I8
    else:
        a = (torch.randn((m, k), device="cuda", generator=g) * 8).to(torch.float8_e4m3fn).view(torch.uint8)
        b = (torch.randn((n, k), device="cuda", generator=g) * 8).to(torch.float8_e4m3fn).view(torch.uint8)
        t = L.E4M3
    a[300:310] = 0                                                   # zero rows: tile scale 0, zero output
    m_live = 500
    rope = None
    if use_rope:
        ang = torch.rand((m, 64), device="cuda", generator=g) * 6.28
        rope = torch.stack([torch.cos(ang), torch.sin(ang)], dim=2).reshape(m, 128).contiguous()
    alpha = 0.37
    raw = torch.empty((m, n), dtype=torch.float32, device="cuda")
    lib.gemm_nt(a, b, raw, t, L.F32, alpha=alpha, m_live=m_live, tile_config=1)
    want = torch.full((m, n), 7, dtype=torch.int16, device="cuda")
    want_sc = torch.full((n // 128, m), -1.0, device="cuda")
    L.call("ts2_row_tile_normalize_rope", m_live, m, raw, L.F32, 1.0, int(normalize), 1 / 24.0, rope, want, want_sc if normalize else None)
    wf = want.view(torch.bfloat16).float()
    # one bf16 ulp, plus a few fp32 ulps of the rotation's operands: own*cos - other*sin can cancel to far below either product, and
    # the two paths round the tile sum (hence the products) differently in the last fp32 bit
    tile_max = wf.abs().view(m, n // 128, 128).amax(2, keepdim=True).expand(m, n // 128, 128).reshape(m, n)
    tol = wf.abs() * 2.0 ** -7 + tile_max * 2.0 ** -21 + 1e-30
    # the 256x256 tile (a wave holds a whole 128-column tile); e4m3 also the 128x128 tile (two waves share a tile's sums), alone and as
    # the expert-grouped product (here every row tile names the one slab)
    one_slab = dict(tile_group=torch.zeros(m // 128, dtype=torch.int32, device="cuda"), b_slab_bytes=n * k)
    for cfg, extra in ((1, {}),) + (((2, {}), (2, one_slab)) if ab != "i8" else ()):
        got = torch.full((m, n), 9, dtype=torch.int16, device="cuda")
        got_sc = torch.full((n // 128, m), -2.0, device="cuda")
        lib.gemm_nt(a, b, got, t, L.BF16, alpha=alpha, m_live=m_live, tile_config=cfg, epilogue=L.EPI_ROW_TILE_NORM, normalize=normalize,
                    vec_scale=1 / 24.0, rope=rope, tile_scale=got_sc if normalize else None, n=n, **extra)
        torch.cuda.synchronize()
        gf = got.view(torch.bfloat16).float()
        assert (gf[m_live:] == 0).all() and (gf[300:310] == 0).all()
        assert ((gf - wf).abs() <= tol).all(), cfg
        assert (gf == wf).float().mean() > 0.99
        if normalize:
            assert torch.allclose(got_sc[:, :m_live], want_sc[:, :m_live], rtol=1e-6, atol=0)
            assert (got_sc[:, 300:310] == 0).all()
    # int8 operands: unsupported with 128x128 tiles, the caller falls back to the two-pass path
    if ab == "i8":
        assert lib.gemm_nt(a, b, got, t, L.BF16, tile_config=2, epilogue=L.EPI_ROW_TILE_NORM, normalize=True, vec_scale=1.0, tile_scale=got_sc,
                           check=False) == -3


@pytest.mark.parametrize("ab,add", [("e4m3", False), ("e4m3", True), ("bf16", True)])
def test_several_products_into_one_result(ab, add):
    """extraSegments: C (+)= sum_i alpha_i * s_i * A_i B_i^T in one launch against the same products launched one after the other
    (store, then accumulate).  The sums are the same fp32 MFMA sums; the one-launch form rescales them in registers between products
    and rounds the total once, so the results agree to a few fp32 ulps of the largest partial sum."""
    print("case several products", ab, add, flush=True)
    from tscale2_amd import lib as L
    lib = L.load()
    m, n, k, nseg = 512, 768, 384, 4
    g = torch.Generator(device="cuda").manual_seed(11)
    As, Bs, alphas, ptrs = [], [], [], []
    for i in range(nseg):
        if ab == "e4m3":
            a = (torch.randn((m, k), device="cuda", generator=g) * 6).to(torch.float8_e4m3fn).view(torch.uint8)
            b = (torch.randn((n, k), device="cuda", generator=g) * 6).to(torch.float8_e4m3fn).view(torch.uint8)
            t = L.E4M3
        else:
            a = torch.randn((m, k), device="cuda", generator=g).bfloat16().view(torch.int16)
            b = torch.randn((n, k), device="cuda", generator=g).bfloat16().view(torch.int16)
            t = L.BF16
        As.append(a); Bs.append(b)
        alphas.append(0.25 * (i + 1))
        ptrs.append(None if i == 2 else torch.full((1,), 0.5 + 0.37 * i, device="cuda"))
    c0 = torch.randn((m, n), device="cuda", generator=g)
    want = c0.clone() if add else torch.empty_like(c0)
    for i in range(nseg):
        lib.gemm_nt(As[i], Bs[i], want, t, L.F32, alpha=alphas[i], alpha_ptr=ptrs[i], tile_config=1,
                    epilogue=L.EPI_ADD if (add or i > 0) else L.EPI_STORE, m_live=500)
    got = c0.clone() if add else torch.full_like(c0, 3.0)
    lib.gemm_nt(As[0], Bs[0], got, t, L.F32, alpha=alphas[0], alpha_ptr=ptrs[0], epilogue=L.EPI_ADD if add else L.EPI_STORE, m_live=500,
                segments=[(As[i], Bs[i], alphas[i], ptrs[i]) for i in range(1, nseg)])
    torch.cuda.synchronize()
    scale = want[:500].abs().max().item()
    assert (got[:500] - want[:500]).abs().max().item() <= 4e-6 * scale
    if not add:
        assert (got[500:] == 0).all()
    # not available for int8 operands; the 128x128 tile takes one further product, not two
    a8 = torch.zeros((m, k), dtype=torch.int8, device="cuda"); b8 = torch.zeros((n, k), dtype=torch.int8, device="cuda")
    assert lib.gemm_nt(a8, b8, got, L.I8, L.F32, segments=[(a8, b8, 1.0, None)], check=False) == -3
    assert lib.gemm_nt(As[0], Bs[0], got, t, L.F32, tile_config=2, segments=[(As[1], Bs[1], 1.0, None), (As[2], Bs[2], 1.0, None)],
                       check=False) == -3


@pytest.mark.parametrize("grouped", [False, True])
@pytest.mark.parametrize("c_type", ["f32", "bf16"])
def test_two_products_into_one_result_on_the_small_tile(grouped, c_type):
    """One further product on the 128x128 tile, plain and with a weight slab per 128-row tile (the expert-grouped dX of two matrices
    that share their rows): against the two products launched one after the other (store, then accumulate).  Same MFMA sums; the
    one-launch form rescales the first in registers and rounds the total once."""
    print("case two products small tile", grouped, c_type, flush=True)
    from tscale2_amd import lib as L
    lib = L.load()
    m, n, k, slabs = 640, 384, 256, 3
    g = torch.Generator(device="cuda").manual_seed(12)
    mk = lambda r, c: (torch.randn((r, c), device="cuda", generator=g) * 6).to(torch.float8_e4m3fn).view(torch.uint8)
    a0, a1 = mk(m, k), mk(m, k)
    b0, b1 = mk(n * (slabs if grouped else 1), k), mk(n * (slabs if grouped else 1), k)
    p0 = torch.full((1,), 0.7, device="cuda")
    kw = dict(n=n)
    if grouped:
        kw.update(tile_group=torch.tensor([2, 0, -1, 1, 2], dtype=torch.int32, device="cuda"), b_slab_bytes=n * k)
    else:
        kw.update(tile_config=2)
    ct, dt = (L.F32, torch.float32) if c_type == "f32" else (L.BF16, torch.bfloat16)
    view = (lambda x: x) if c_type == "f32" else (lambda x: x.view(torch.int16))
    want = torch.full((m, n), 3.0, dtype=torch.float32, device="cuda")
    lib.gemm_nt(a0, b0, want, L.E4M3, L.F32, alpha=0.25, alpha_ptr=p0, **kw)
    lib.gemm_nt(a1, b1, want, L.E4M3, L.F32, alpha=0.5, epilogue=L.EPI_ADD, **kw)
    got = torch.full((m, n), 3.0, dtype=dt, device="cuda")
    lib.gemm_nt(a0, b0, view(got), L.E4M3, ct, alpha=0.25, alpha_ptr=p0, segments=[(a1, b1, 0.5, None)], **kw)
    torch.cuda.synchronize()
    scale = want.abs().max().item()
    tol = 4e-6 * scale if c_type == "f32" else 2.0 ** -8 * scale
    assert (got.float() - want).abs().max().item() <= tol
    if grouped:
        assert (got[256:384].float() == 3.0).all()   # the skipped tile is left alone


@pytest.mark.parametrize("ab,tile", [("e4m3", 1), ("i8", 1), ("e4m3", 2)])
def test_half_results_are_the_rounded_fp32_results(ab, tile):
    """cType TS2_F16 (the final layer's logits): every element is the fp32 result of the same launch configuration rounded to the
    nearest IEEE half; rows >= mLive are zero."""
    print("case half results", ab, tile, flush=True)
    from tscale2_amd import lib as L
    lib = L.load()
    m, n, k = 512, 768, 256
    g = torch.Generator(device="cuda").manual_seed(17)
    if ab == "i8":
        a = torch.randint(-100, 100, (m, k), dtype=torch.int8, device="cuda", generator=g)
        b = torch.randint(-100, 100, (n, k), dtype=torch.int8, device="cuda", generator=g)
        t = L.I8
    else:
        a = (torch.randn((m, k), device="cuda", generator=g) * 6).to(torch.float8_e4m3fn).view(torch.uint8)
        b = (torch.randn((n, k), device="cuda", generator=g) * 6).to(torch.float8_e4m3fn).view(torch.uint8)
        t = L.E4M3
    c32 = torch.empty((m, n), dtype=torch.float32, device="cuda")
    c16 = torch.full((m, n), 7, dtype=torch.int16, device="cuda")
    lib.gemm_nt(a, b, c32, t, L.F32, alpha=3e-3, tile_config=tile, m_live=500)
    lib.gemm_nt(a, b, c16, t, L.F16, alpha=3e-3, tile_config=tile, m_live=500)
    torch.cuda.synchronize()
    assert torch.equal(c16.view(torch.float16), c32.half())
    assert (c16[500:] == 0).all()
    assert lib.gemm_nt(a, b, c16, t, L.F16, epilogue=L.EPI_ADD, check=False) == -3


@pytest.mark.parametrize("cfg", [0, 1, 2])
def test_products_per_group_of_contraction_rows_are_bit_exact(lib, orc, cfg):
    """The per-expert delta mode: one product per group g over the contraction range groupOffsets[g] .. groupOffsets[g+1], written
    to its own slab of C.  int8 operands with the int32 result must equal the oracle's product over that range, on the 128x128 and on
    the 256x256 tile (cfg 0 lets the library choose: with the groups counted, 256x256 here); an empty group gives a zero slab."""
    print(f"case grouped contraction cfg={cfg}", flush=True)
    from tscale2_amd import lib as L
    r = np.random.default_rng(40 + cfg)
    m, n, k = 256, 512, 1792
    offs = np.array([0, 384, 384, 1280, 1792], np.int32)          # group 1 is empty
    groups = len(offs) - 1
    a = r.integers(-128, 128, (m, k), dtype=np.int8)
    b = r.integers(-128, 128, (n, k), dtype=np.int8)
    tc = torch.full((groups * m, n), -7, dtype=torch.int32, device="cuda")
    lib.gemm_nt(torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), tc, L.I8, L.I32, tile_config=cfg, m=m,
                group_offsets=torch.from_numpy(offs).cuda(), groups=groups, c_slab_bytes=m * n * 4)
    torch.cuda.synchronize()
    got = tc.cpu().numpy().reshape(groups, m, n)
    for g in range(groups):
        lo, hi = int(offs[g]), int(offs[g + 1])
        want = orc_gemm_i8(orc, np.ascontiguousarray(a[:, lo:hi]), np.ascontiguousarray(b[:, lo:hi])) if hi > lo else np.zeros((m, n), np.int32)
        assert np.array_equal(got[g], want), g


def test_weight_slab_chosen_per_row_tile_is_bit_exact(lib, orc):
    """The expert-grouped forward / dX mode: every 128-row tile of A multiplies the B slab its tileGroup entry names; tiles with -1
    are skipped and leave C alone."""
    print("case slab per row tile", flush=True)
    from tscale2_amd import lib as L
    r = np.random.default_rng(44)
    m, n, k, slabs = 640, 256, 512, 3
    tg = np.array([2, 0, -1, 1, 2], np.int32)
    a = r.integers(-128, 128, (m, k), dtype=np.int8)
    b = r.integers(-128, 128, (slabs * n, k), dtype=np.int8)
    tc = torch.full((m, n), -7, dtype=torch.int32, device="cuda")
    lib.gemm_nt(torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), tc, L.I8, L.I32, n=n,
                tile_group=torch.from_numpy(tg).cuda(), b_slab_bytes=n * k)
    torch.cuda.synchronize()
    got = tc.cpu().numpy()
    for t, g in enumerate(tg):
        rows = slice(t * 128, (t + 1) * 128)
        if g < 0:
            assert np.all(got[rows] == -7)
        else:
            assert np.array_equal(got[rows], orc_gemm_i8(orc, np.ascontiguousarray(a[rows]), np.ascontiguousarray(b[g * n:(g + 1) * n])))


@pytest.mark.parametrize("n,k,shrink,c16", [(512, 1024, 1, "bf16"), (1024, 512, 2, "bf16"), (256, 640, 0, "f16"), (512, 2048, 2, "bf16")])
def test_grouped_products_on_the_persistent_kernel(lib, n, k, shrink, c16):
    """The expert-grouped e4m3 product with a 16-bit result on the persistent kernel (operands exchanged: a tile is 256 result columns
    of one expert x the 128 tokens of a row tile): bit-identical to the 128x128 kernels (same contraction order per accumulator), tiles
    without an expert leave C alone, rows from mLive on are zeros, per-token row scales.  shrink > 0 runs many tiles per workgroup
    (the roles of the wave groups alternate, the operand ring wraps around tile boundaries)."""
    print(f"case grouped persistent n={n} k={k} shrink={shrink} {c16}", flush=True)
    from tscale2_amd import lib as L
    g = torch.Generator(device="cuda").manual_seed(100 + n + k)
    slabs, tiles = 5, 23
    m = tiles * 128
    r = np.random.default_rng(n + k)
    tg = r.integers(0, slabs, tiles).astype(np.int32)
    tg[[3, 11, 22]] = -1
    tg[0], tg[1] = 4, 0
    a = (torch.randn((m, k), device="cuda", generator=g) * 4).to(torch.float8_e4m3fn).view(torch.uint8)
    b = (torch.randn((slabs * n, k), device="cuda", generator=g) * 4).to(torch.float8_e4m3fn).view(torch.uint8)
    rs = torch.rand((m,), device="cuda", generator=g) + 0.5
    ct = L.F16 if c16 == "f16" else L.BF16
    tgd = torch.from_numpy(tg).cuda()
    m_live = m - 128 - 37  # inside the last tile that has an expert
    res = []
    for cfg in (32768, 4096 | (shrink << 13)):
        c = torch.full((m, n), 0x1234, dtype=torch.int16, device="cuda")
        lib.gemm_nt(a, b, c, L.E4M3, ct, alpha=2e-3, row_scale=rs, n=n, tile_group=tgd, b_slab_bytes=n * k, m_live=m_live, tile_config=cfg)
        torch.cuda.synchronize()
        res.append(c)
    old, new = res
    assert torch.equal(old, new)
    for t, e in enumerate(tg):
        rows = new[t * 128:(t + 1) * 128]
        if e < 0:
            assert (rows == 0x1234).all(), t
    assert (new[m_live:m - 128] == 0).all()
    # and against the product itself on one tile
    t = 1
    view = torch.float16 if c16 == "f16" else torch.bfloat16
    af = a[t * 128:(t + 1) * 128].view(torch.float8_e4m3fn).float()
    bf = b[tg[t] * n:(tg[t] + 1) * n].view(torch.float8_e4m3fn).float()
    want = (af @ bf.T) * 2e-3 * rs[t * 128:(t + 1) * 128, None]
    assert torch.allclose(new[t * 128:(t + 1) * 128].view(view).float(), want, rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("n,k,tiles,shrink,with_rope", [(512, 1024, 23, 1, False), (256, 512, 9, 2, False), (1024, 640, 8, 2, True), (256, 1024, 1, 0, False)])
def test_grouped_normalised_products_on_the_persistent_kernel(lib, n, k, tiles, shrink, with_rope):
    """The expert-grouped product with the row-tile normalising epilogue (the experts' expand product) on the persistent kernel: a
    token's 128-column tile is held by two waves, which exchange their sums of squares through LDS.  Normalised bf16 rows and tile
    scales bit-identical to the 128x128 kernel's, with and without the rotation of column pairs; odd and even numbers of tiles per
    workgroup (either wave group ends the list)."""
    print(f"case grouped persistent normalised n={n} k={k} tiles={tiles} shrink={shrink}", flush=True)
    from tscale2_amd import lib as L
    g = torch.Generator(device="cuda").manual_seed(300 + n + k + tiles)
    slabs = 3
    m = tiles * 128
    tg = (np.arange(tiles) * 7 % slabs).astype(np.int32)
    if tiles > 4:
        tg[4] = -1
    a = (torch.randn((m, k), device="cuda", generator=g) * 4).to(torch.float8_e4m3fn).view(torch.uint8)
    b = (torch.randn((slabs * n, k), device="cuda", generator=g) * 4).to(torch.float8_e4m3fn).view(torch.uint8)
    tgd = torch.from_numpy(tg).cuda()
    m_live = m - 50 if tg[-1] >= 0 else m
    rope = None
    if with_rope:   # (cos, sin) pairs per row and column pair of a 128-wide tile
        ang = torch.rand((m, 64), device="cuda", generator=g) * 6.28
        rope = torch.stack((ang.cos(), ang.sin()), dim=2).reshape(m, 128).contiguous()
    res = []
    for cfg in (32768, 4096 | (shrink << 13)):
        c = torch.full((m, n), 0x1234, dtype=torch.int16, device="cuda")
        ts = torch.full((n // 128, m), -3.0, device="cuda")
        lib.gemm_nt(a, b, c, L.E4M3, L.BF16, alpha=2e-3, n=n, tile_group=tgd, b_slab_bytes=n * k, m_live=m_live, tile_config=cfg,
                    epilogue=L.EPI_ROW_TILE_NORM, normalize=True, vec_scale=1 / 24.0, tile_scale=ts, rope=rope)
        torch.cuda.synchronize()
        res.append((c, ts))
    assert torch.equal(res[0][0], res[1][0])
    assert torch.equal(res[0][1], res[1][1])
    c, ts = res[1]
    if tiles > 4:
        assert (c[4 * 128:5 * 128] == 0x1234).all() and (ts[:, 4 * 128:5 * 128] == -3.0).all()
    # normalised: mean square of a tile = (1 / vecScale)^2
    t = 1 if tiles > 1 else 0
    x = c[t * 128:t * 128 + 64].view(torch.bfloat16).float().view(64, n // 128, 128)
    assert torch.allclose((x * x).mean(2), torch.full((64, n // 128), 576.0, device="cuda"), rtol=2e-2)


@pytest.mark.parametrize("f0,f1", [(0.7, 0.3), (0.5, 0.5), (0.9, 0.0), (0.0, 0.4)])
def test_grouped_sum_of_two_products_on_the_persistent_kernel(lib, f0, f1):
    """C = alpha (f0 A0 B0_g^T + f1 A1 B1_g^T) per expert-grouped row tile (the dX of an expert's expand and gate matrices): the persistent
    kernel runs the second product's steps behind the first's and rescales the accumulators at the seam, like the two-product form of
    the 128x128 kernel - bit-identical to it, also with a zero factor on either product"""
    print(f"case grouped two products {f0} {f1}", flush=True)
    from tscale2_amd import lib as L
    g = torch.Generator(device="cuda").manual_seed(7)
    slabs, tiles, n, k = 4, 19, 512, 512
    m = tiles * 128
    tg = (np.arange(tiles) % slabs).astype(np.int32)
    tg[5] = -1
    mk = lambda r, c: (torch.randn((r, c), device="cuda", generator=g) * 4).to(torch.float8_e4m3fn).view(torch.uint8)
    a0, a1, b0, b1 = mk(m, k), mk(m, k), mk(slabs * n, k), mk(slabs * n, k)
    p0, p1 = torch.full((1,), f0, device="cuda"), torch.full((1,), f1, device="cuda")
    tgd = torch.from_numpy(tg).cuda()
    res = []
    for cfg in (32768, 4096 | (2 << 13)):
        c = torch.full((m, n), 0x1234, dtype=torch.int16, device="cuda")
        lib.gemm_nt(a0, b0, c, L.E4M3, L.BF16, alpha=3e-3, alpha_ptr=p0, n=n, tile_group=tgd, b_slab_bytes=n * k, tile_config=cfg,
                    segments=((a1, b1, 3e-3, p1),))
        torch.cuda.synchronize()
        res.append(c)
    assert torch.equal(res[0], res[1])
    assert (res[1][5 * 128:6 * 128] == 0x1234).all()
    t = 2
    rows = slice(t * 128, (t + 1) * 128)
    f = lambda x: x.view(torch.float8_e4m3fn).float()
    want = 3e-3 * (f0 * f(a0[rows]) @ f(b0[tg[t] * n:(tg[t] + 1) * n]).T + f1 * f(a1[rows]) @ f(b1[tg[t] * n:(tg[t] + 1) * n]).T)
    assert torch.allclose(res[1][rows].view(torch.bfloat16).float(), want, rtol=1e-2, atol=2e-3)


@pytest.mark.parametrize("zero_at", [(0,), (1,), (3,), (1, 2), (0, 1, 2, 3)])
def test_products_with_a_zero_factor_contribute_nothing(zero_at):
    """a device-resident factor of zero (the scale of an all-zero matrix) on any of the products of a one-launch sum: the product is
    skipped, the others keep their sum - no 0 * inf from rescaling to a zero factor"""
    print("case several products, zero factors at", zero_at, flush=True)
    from tscale2_amd import lib as L
    lib = L.load()
    m, n, k, nseg = 512, 512, 256, 4
    g = torch.Generator(device="cuda").manual_seed(13)
    mk = lambda r, c: (torch.randn((r, c), device="cuda", generator=g) * 6).to(torch.float8_e4m3fn).view(torch.uint8)
    As = [mk(m, k) for _ in range(nseg)]; Bs = [mk(n, k) for _ in range(nseg)]
    ptrs = [torch.full((1,), 0.0 if i in zero_at else 0.5 + 0.3 * i, device="cuda") for i in range(nseg)]
    want = torch.zeros((m, n), device="cuda")
    for i in range(nseg):
        lib.gemm_nt(As[i], Bs[i], want, L.E4M3, L.F32, alpha=0.25, alpha_ptr=ptrs[i], tile_config=1, epilogue=L.EPI_ADD)
    got = torch.full((m, n), 3.0, device="cuda")
    lib.gemm_nt(As[0], Bs[0], got, L.E4M3, L.F32, alpha=0.25, alpha_ptr=ptrs[0], segments=[(As[i], Bs[i], 0.25, ptrs[i]) for i in range(1, nseg)])
    torch.cuda.synchronize()
    assert torch.isfinite(got).all()
    assert (got - want).abs().max().item() <= 4e-6 * max(want.abs().max().item(), 1e-30)
    # the 128x128 tile with one further product
    for za in ((0,), (1,), (0, 1)):
        p2 = [torch.full((1,), 0.0 if i in za else 0.7, device="cuda") for i in range(2)]
        want2 = torch.zeros((m, n), device="cuda")
        for i in range(2):
            lib.gemm_nt(As[i], Bs[i], want2, L.E4M3, L.F32, alpha=0.5, alpha_ptr=p2[i], tile_config=2, epilogue=L.EPI_ADD)
        got2 = torch.full((m, n), 3.0, device="cuda")
        lib.gemm_nt(As[0], Bs[0], got2, L.E4M3, L.F32, alpha=0.5, alpha_ptr=p2[0], tile_config=2, segments=[(As[1], Bs[1], 0.5, p2[1])])
        torch.cuda.synchronize()
        assert torch.isfinite(got2).all() and (got2 - want2).abs().max().item() <= 4e-6 * max(want2.abs().max().item(), 1e-30), za


def test_contraction_major_bf16_operands_equal_the_transposed_product(lib):
    """kMajor with bf16 operands (the delta of the final layer: gradient [token][vocab] and final state [token][dim] as they lie, the
    reference's Fp16MatMul<1, 1, TStoreDelta>, src/gpt/compute/gpu_final.cuh:265): bit-identical to the product of the explicitly
    transposed operands, for the fp32 store, the packed delta and stored slices; strided views, 9 contraction steps."""
    print("case contraction-major bf16 operands", flush=True)
    from tscale2_amd import lib as L
    m, n, k = 512, 768, 576
    g = torch.Generator(device="cuda").manual_seed(32)
    big_a = torch.randn((k, m + 256), device="cuda", generator=g).bfloat16()
    big_b = torch.randn((k, n + 512), device="cuda", generator=g).bfloat16()
    akm, bkn = big_a[:, 128:128 + m], big_b[:, 256:256 + n]      # [k][m], [k][n] views with larger row strides
    at, bt = akm.t().contiguous(), bkn.t().contiguous()
    c0 = torch.zeros((m, n), device="cuda"); c1 = torch.ones((m, n), device="cuda")
    lib.gemm_nt(at, bt, c0, L.BF16, L.F32, alpha=0.5, tile_config=1)
    lib.gemm_nt(akm, bkn, c1, L.BF16, L.F32, alpha=0.5, tile_config=1, m=m, n=n, k=k, k_major=True)
    torch.cuda.synchronize()
    assert torch.equal(c0, c1)
    ref = (akm.double().t() @ bkn.double()) * 0.5
    assert float((c1.double() - ref).abs().max()) <= 1e-5 * float(ref.abs().max())
    d0 = torch.zeros((m, n), dtype=torch.int8, device="cuda"); d1 = torch.ones_like(d0)
    t0 = torch.zeros((n // 128, m), device="cuda"); t1 = torch.ones_like(t0)
    lib.gemm_nt(at, bt, d0, L.BF16, L.I8, epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=t0, tile_config=1)
    lib.gemm_nt(akm, bkn, d1, L.BF16, L.I8, epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=t1, tile_config=1, m=m, n=n, k=k, k_major=True)
    torch.cuda.synchronize()
    assert torch.equal(d0, d1) and torch.equal(t0, t1) and int(d1.abs().max()) == 127
    s0 = torch.zeros((3, m, n), device="cuda"); s1 = torch.ones_like(s0)
    lib.gemm_nt(at, bt, s0.view(3 * m, n), L.BF16, L.F32, split_k=3, split_slab_bytes=m * n * 4, tile_config=1, m=m, n=n, k=k)
    lib.gemm_nt(akm, bkn, s1.view(3 * m, n), L.BF16, L.F32, split_k=3, split_slab_bytes=m * n * 4, tile_config=1, m=m, n=n, k=k, k_major=True)
    torch.cuda.synchronize()
    assert torch.equal(s0, s1)
    assert float((s1.sum(0).double() - ref * 2).abs().max()) <= 1e-5 * float(ref.abs().max()) * 2


def test_ring_pipeline_on_the_small_tile_equals_the_two_stage_loop(lib):
    """The 128x128 tile has two kernels for e4m3 operands: the two-stage loop and the ring pipeline (three A and two B stages, two
    workgroups per CU), chosen by the contraction length (tileConfig bit 7 / bit 4 force one or the other).  Both feed the MFMAs the
    same operands in the same order, so every result type must come out bit-identical: fp32 stored and accumulated (contractions of
    1 .. 16 steps, live rows short of m), bf16, the packed delta, the normalising epilogue, the expert-grouped product with a skipped
    row tile, and two grouped products into one result."""
    print("case small-tile ring", flush=True)
    from tscale2_amd import lib as L
    RING, LOOP = 2 | 128, 2 | 16
    g = torch.Generator(device="cuda").manual_seed(3)

    def codes(shape):  # e4m3 bytes without the NaN codes, both signs
        return (torch.randint(0, 120, shape, device="cuda", generator=g) | (torch.randint(0, 2, shape, device="cuda", generator=g) << 7)).to(torch.uint8)

    def both(fn, outs, skip_rows=None, loop=LOOP):
        res = []
        for cfg, fill in ((loop, 0), (RING, 1)):
            for o in outs:
                o.fill_(fill)
            fn(cfg)
            torch.cuda.synchronize()
            res.append([o.clone() for o in outs])
        for a, b in zip(*res):
            if skip_rows is not None:   # rows of a skipped tile keep what the buffer held
                a[skip_rows] = 0; b[skip_rows] = 0
            assert torch.equal(a, b)
        assert float(res[0][0].float().abs().max()) > 0
    for k in (128, 256, 384, 768, 1152, 2048):
        m, n = 384, 256
        a, b = codes((m, k)), codes((n, k))
        c = torch.zeros((m, n), device="cuda")
        both(lambda cfg: lib.gemm_nt(a, b, c, L.E4M3, L.F32, alpha=0.25, tile_config=cfg, m_live=300), [c])
    m, n, k = 640, 384, 896
    a, b = codes((m, k)), codes((n, k))
    c16 = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    both(lambda cfg: lib.gemm_nt(a, b, c16, L.E4M3, L.BF16, alpha=0.25, tile_config=cfg), [c16])
    c32 = torch.zeros((m, n), device="cuda")
    lib.gemm_nt(a, b, c32, L.E4M3, L.F32, alpha=0.25, tile_config=LOOP)
    torch.cuda.synchronize()
    assert torch.equal(c16, c32.bfloat16())  # and both are the rounded fp32 result (which leaves through another epilogue)
    # live rows short of m, and a result whose rows start on 4-byte, not 16-byte, boundaries (the ring's 16-bit rows leave through LDS as
    # 16-byte stores when they can)
    both(lambda cfg: lib.gemm_nt(a, b, c16, L.E4M3, L.BF16, alpha=0.25, tile_config=cfg, m_live=500), [c16])
    wide16 = torch.zeros((m, n + 2), dtype=torch.bfloat16, device="cuda")
    wide16[:, n:] = 7
    both(lambda cfg: lib.gemm_nt(a, b, wide16[:, :n], L.E4M3, L.BF16, alpha=0.25, tile_config=cfg), [wide16[:, :n]])
    assert bool((wide16[:, n:] == 7).all())  # nothing written past the row's end
    h16 = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    both(lambda cfg: lib.gemm_nt(a, b, h16, L.E4M3, L.F16, alpha=0.25, tile_config=cfg), [h16])
    cadd = torch.zeros((m, n), device="cuda")
    start = torch.randn((m, n), device="cuda", generator=g)

    def add(cfg):
        cadd.copy_(start)
        lib.gemm_nt(a, b, cadd, L.E4M3, L.F32, alpha=0.25, tile_config=cfg, epilogue=L.EPI_ADD)
    both(add, [cadd])
    d8 = torch.zeros((m, n), dtype=torch.int8, device="cuda"); ts = torch.zeros((n // 128, m), device="cuda")
    both(lambda cfg: lib.gemm_nt(a, b, d8, L.E4M3, L.I8, tile_config=cfg, epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=ts), [d8, ts])
    cn = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda"); tn = torch.zeros((n // 128, m), device="cuda")
    both(lambda cfg: lib.gemm_nt(a, b, cn, L.E4M3, L.BF16, alpha=0.3, tile_config=cfg, epilogue=L.EPI_ROW_TILE_NORM, normalize=True,
                                 vec_scale=1 / 24.0, tile_scale=tn), [cn, tn])
    slabs = 3
    bs = codes((slabs * n, k))
    tg = torch.tensor([2, 0, -1, 1, 2], dtype=torch.int32, device="cuda")
    cg = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    skipped = slice(256, 384)
    both(lambda cfg: lib.gemm_nt(a, bs, cg, L.E4M3, L.BF16, n=n, tile_config=cfg, tile_group=tg, b_slab_bytes=n * k), [cg], skipped)
    a2, bs2 = codes((m, k)), codes((slabs * n, k))
    sc1 = torch.tensor([0.7], device="cuda"); sc2 = torch.tensor([1.9], device="cuda")
    both(lambda cfg: lib.gemm_nt(a, bs, cg, L.E4M3, L.BF16, n=n, alpha=0.1, alpha_ptr=sc1, tile_config=cfg, tile_group=tg, b_slab_bytes=n * k,
                                 segments=[(a2, bs2, 0.1, sc2)]), [cg], skipped, loop=2)  # (k < 1024: the loop is the library's choice)
    # the grouped product against a plain product per row tile
    want = torch.zeros((m, n), device="cuda")
    for t, e in enumerate(tg.tolist()):
        if e >= 0:
            lib.gemm_nt(a[t * 128:(t + 1) * 128], bs[e * n:(e + 1) * n], want[t * 128:(t + 1) * 128], L.E4M3, L.F32, tile_config=LOOP)
    got = torch.zeros((m, n), device="cuda")
    lib.gemm_nt(a, bs, got, L.E4M3, L.F32, n=n, tile_config=RING, tile_group=tg, b_slab_bytes=n * k)
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_contraction_major_operands_equal_the_transposed_product(lib, orc):
    """kMajor: A [k][m], B [k][n] (the untransposed activations of a delta product) against the same product on explicitly transposed
    operands.  Both feed the MFMAs the same operand bytes in the same contraction slots, so fp32 results, stored slices and packed
    deltas must be bit-identical; operands with live strides larger than the tile, a contraction of 9 steps (ring loop + tail)"""
    print("case contraction-major operands", flush=True)
    from tscale2_amd import lib as L
    m, n, k = 512, 768, 1152
    r = np.random.default_rng(31)

    def codes(shape):  # e4m3 bytes without the NaN codes, both signs
        return (r.integers(0, 120, shape) | (r.integers(0, 2, shape) << 7)).astype(np.uint8)
    big_a, big_b = codes((k, m + 256)), codes((k, n + 512))
    akm = torch.from_numpy(big_a).cuda()[:, 128:128 + m]   # [k][m] view with a larger row stride
    bkn = torch.from_numpy(big_b).cuda()[:, 256:256 + n]
    at, bt = akm.t().contiguous(), bkn.t().contiguous()    # [m][k], [n][k]
    # fp32 store
    c0 = torch.zeros((m, n), device="cuda"); c1 = torch.ones((m, n), device="cuda")
    lib.gemm_nt(at, bt, c0, L.E4M3, L.F32, alpha=0.5, tile_config=1)
    lib.gemm_nt(akm, bkn, c1, L.E4M3, L.F32, alpha=0.5, tile_config=1, m=m, n=n, k=k, k_major=True)
    torch.cuda.synchronize()
    assert torch.equal(c0, c1) and float(c0.abs().max()) > 0
    tab = orc.e4m3_table(hw=True)
    ref = (tab[big_a[:, 128:128 + m]].astype(np.float64).T @ tab[big_b[:, 256:256 + n]].astype(np.float64)) * 0.5
    assert np.abs(c1.cpu().numpy() - ref).max() <= 2e-4 * np.abs(ref).max()
    # packed delta
    d0 = torch.zeros((m, n), dtype=torch.int8, device="cuda"); d1 = torch.ones_like(d0)
    t0 = torch.zeros((n // 128, m), device="cuda"); t1 = torch.ones_like(t0)
    lib.gemm_nt(at, bt, d0, L.E4M3, L.I8, epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=t0, tile_config=1)
    lib.gemm_nt(akm, bkn, d1, L.E4M3, L.I8, epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=t1, tile_config=1, m=m, n=n, k=k, k_major=True)
    torch.cuda.synchronize()
    assert torch.equal(d0, d1) and torch.equal(t0, t1)
    # three stored slices of the contraction
    s0 = torch.zeros((3, m, n), device="cuda"); s1 = torch.ones_like(s0)
    lib.gemm_nt(at, bt, s0.view(3 * m, n), L.E4M3, L.F32, split_k=3, split_slab_bytes=m * n * 4, tile_config=1, m=m, n=n, k=k)
    lib.gemm_nt(akm, bkn, s1.view(3 * m, n), L.E4M3, L.F32, split_k=3, split_slab_bytes=m * n * 4, tile_config=1, m=m, n=n, k=k, k_major=True)
    torch.cuda.synchronize()
    assert torch.equal(s0, s1)
    assert np.abs(s1.sum(0).cpu().numpy() - ref * 2).max() <= 2e-4 * np.abs(ref).max() * 2
    # one packed delta per group of contraction rows (the per-expert deltas; group 1 is empty, group 0 a single step)
    offs = torch.tensor([0, 128, 128, 768, 1152], dtype=torch.int32, device="cuda")
    g0 = torch.zeros((4 * m, n), dtype=torch.int8, device="cuda"); g1 = torch.ones_like(g0)
    u0 = torch.zeros((n // 128, 4 * m), device="cuda"); u1 = torch.ones_like(u0)
    kw = dict(epilogue=L.EPI_ROW_TILE_MAXNORM, tile_config=1, m=m, n=n, k=k, group_offsets=offs, groups=4, c_slab_bytes=m * n,
              tile_scale_slab_bytes=m * 4)
    lib.gemm_nt(at, bt, g0, L.E4M3, L.I8, tile_scale=u0, **kw)
    lib.gemm_nt(akm, bkn, g1, L.E4M3, L.I8, tile_scale=u1, k_major=True, **kw)
    torch.cuda.synchronize()
    assert torch.equal(g0, g1) and torch.equal(u0, u1) and int(g1[:m].abs().max()) > 0 and int(g1[m:2 * m].abs().max()) == 0
    # what the variant does not take
    TS2_ERR_UNSUPPORTED = -3
    ai = torch.zeros((k, m), dtype=torch.int8, device="cuda"); bi = torch.zeros((k, n), dtype=torch.int8, device="cuda")
    ci = torch.zeros((m, n), dtype=torch.int32, device="cuda")
    assert lib.gemm_nt(ai, bi, ci, L.I8, L.I32, m=m, n=n, k=k, k_major=True, check=False) == TS2_ERR_UNSUPPORTED
