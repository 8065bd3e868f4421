"""GPU parity of the persistent eight-wave GEMM kernel whose epilogue runs under the next tile's main loop (tileConfig bit 12) against
the oracle (int8, bit-exact) and against the 256x256 ring kernel, whose own parity tests are in test_gemm_gpu.py: the kernels add the
same products in the same order per accumulator, so every result type must agree bit for bit.  Bits 13-14 of tileConfig shrink the
number of workgroups, so that small products walk through many tiles per workgroup (both wave groups, odd and even tile counts)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from oracle_lib import Oracle, _ptr  # noqa: E402

PING = 4096


def shrink(n):
    return n << 13


@pytest.fixture(scope="module")
def lib():
    import tscale2_amd
    return tscale2_amd.load()


@pytest.fixture(scope="module")
def orc():
    return Oracle()


def _e4m3(shape, g, scale=6.0):
    return (torch.randn(shape, device="cuda", generator=g) * scale).to(torch.float8_e4m3fn).view(torch.uint8)


# (m, n, k, shrink): tiles = (m/256)*(n/128) over 256 >> 2*shrink workgroups (at least 8)
@pytest.mark.parametrize("m,n,k,sh", [(256, 128, 1024, 0), (512, 256, 1024, 3), (256, 384, 1152, 3), (768, 640, 1280, 3), (1024, 1152, 1408, 2),
                                      (2048, 2560, 1024, 1), (256, 128, 4096, 0)])
def test_int8_int32_sums_are_exact(lib, orc, m, n, k, sh):
    print(f"case ping int8 exact m={m} n={n} k={k} shrink={sh}", flush=True)
    from tscale2_amd import lib as L
    r = np.random.default_rng(m + n + k)
    a = r.integers(-128, 128, (m, k), dtype=np.int8)
    b = r.integers(-128, 128, (n, k), dtype=np.int8)
    ref = np.empty((m, n), np.int32)
    orc.lib.orc_gemm_i8_nt(_ptr(a), _ptr(b), _ptr(ref), m, n, k)
    tc = torch.full((m, n), -7, dtype=torch.int32, device="cuda")
    lib.gemm_nt(torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), tc, L.I8, L.I32, tile_config=PING | shrink(sh))
    torch.cuda.synchronize()
    assert np.array_equal(tc.cpu().numpy(), ref)


def test_int8_row_scaled_results_equal_the_ring_kernel(lib):
    print("case ping int8 rowscale", flush=True)
    from tscale2_amd import lib as L
    m, n, k = 1024, 512, 1024
    g = torch.Generator(device="cuda").manual_seed(3)
    a = torch.randint(-127, 128, (m, k), dtype=torch.int8, device="cuda", generator=g)
    b = torch.randint(-127, 128, (n, k), dtype=torch.int8, device="cuda", generator=g)
    rs = torch.rand(m, device="cuda", generator=g) + 0.1
    c0 = torch.randn((m, n), device="cuda", generator=g)
    for epi, m_live in ((L.EPI_STORE, 0), (L.EPI_STORE, 700), (L.EPI_ADD, 0), (L.EPI_ADD, 700)):
        want, got = c0.clone(), c0.clone()
        lib.gemm_nt(a, b, want, L.I8, L.F32, row_scale=rs, alpha=0.01, epilogue=epi, tile_config=1, m_live=m_live)
        lib.gemm_nt(a, b, got, L.I8, L.F32, row_scale=rs, alpha=0.01, epilogue=epi, tile_config=PING | shrink(3), m_live=m_live)
        torch.cuda.synchronize()
        assert torch.equal(got, want), (epi, m_live)


@pytest.mark.parametrize("ab", ["e4m3", "bf16"])
@pytest.mark.parametrize("m,n,k,sh", [(256, 256, 1024, 0), (1024, 768, 1536, 3), (2048, 1280, 2048, 2)])
def test_float_results_equal_the_ring_kernel_bit_for_bit(lib, ab, m, n, k, sh):
    """fp32 store and accumulate, bf16 store and accumulate, IEEE half store; live rows short of m."""
    print(f"case ping float {ab} m={m} n={n} k={k}", flush=True)
    from tscale2_amd import lib as L
    g = torch.Generator(device="cuda").manual_seed(m + k)
    kk = k if ab == "e4m3" else k // 2
    if ab == "e4m3":
        a, b, t = _e4m3((m, kk), g), _e4m3((n, kk), g), L.E4M3
    else:
        a = torch.randn((m, kk), device="cuda", generator=g).bfloat16().view(torch.int16)
        b = torch.randn((n, kk), device="cuda", generator=g).bfloat16().view(torch.int16)
        t = L.BF16
    aptr = torch.full((1,), 0.61, device="cuda")
    c0 = torch.randn((m, n), device="cuda", generator=g)
    for c_type, epi, m_live in ((L.F32, L.EPI_STORE, 0), (L.F32, L.EPI_STORE, m - 37), (L.F32, L.EPI_ADD, m - 37), (L.BF16, L.EPI_STORE, 0),
                                (L.BF16, L.EPI_STORE, m - 37), (L.BF16, L.EPI_ADD, 0), (L.F16, L.EPI_STORE, m - 5)):
        if c_type == L.F32:
            want, got = c0.clone(), c0.clone()
            wv, gv = want, got
        else:
            dt = torch.bfloat16 if c_type == L.BF16 else torch.float16
            want, got = c0.to(dt), c0.to(dt)
            wv, gv = want.view(torch.int16), got.view(torch.int16)
        lib.gemm_nt(a, b, wv, t, c_type, alpha=0.02, alpha_ptr=aptr, epilogue=epi, tile_config=1, m_live=m_live)
        lib.gemm_nt(a, b, gv, t, c_type, alpha=0.02, alpha_ptr=aptr, epilogue=epi, tile_config=PING | shrink(sh), m_live=m_live)
        torch.cuda.synchronize()
        assert torch.equal(gv, wv), (c_type, epi, m_live)
    # 16-bit results whose rows do not start on 16 bytes (a view four columns into a wider array) leave as pairs of columns instead of
    # row segments: same values, neighbours untouched
    for c_type, dt in ((L.BF16, torch.bfloat16), (L.F16, torch.float16)):
        wide = torch.full((m, n + 8), 7.0, device="cuda").to(dt)
        want = torch.empty((m, n), device="cuda").to(dt)
        lib.gemm_nt(a, b, want.view(torch.int16), t, c_type, alpha=0.02, alpha_ptr=aptr, tile_config=1, m_live=m - 37)
        lib.gemm_nt(a, b, wide.view(torch.int16)[:, 4:4 + n], t, c_type, alpha=0.02, alpha_ptr=aptr, tile_config=PING | shrink(sh), m_live=m - 37)
        torch.cuda.synchronize()
        assert torch.equal(wide[:, 4:4 + n].view(torch.int16), want.view(torch.int16)), c_type
        assert bool((wide[:, :4] == 7.0).all()) and bool((wide[:, 4 + n:] == 7.0).all())
    got = torch.empty((m, n), device="cuda")
    lib.gemm_nt(a, b, got, t, L.F32, tile_config=PING | shrink(sh))
    torch.cuda.synchronize()
    if ab == "e4m3":
        fa, fb = a.view(torch.float8_e4m3fn).double(), b.view(torch.float8_e4m3fn).double()
    else:
        fa, fb = a.view(torch.bfloat16).double(), b.view(torch.bfloat16).double()
    ref = fa @ fb.T
    assert (got.double() - ref).abs().max().item() <= 1e-4 * ref.abs().max().item()


def test_calls_the_kernel_cannot_run_are_refused(lib):
    from tscale2_amd import lib as L
    a = torch.zeros((256, 512), dtype=torch.int8, device="cuda")
    b = torch.zeros((128, 512), dtype=torch.int8, device="cuda")
    c = torch.zeros((256, 128), device="cuda")
    assert lib.gemm_nt(a, b, c, L.I8, L.F32, tile_config=PING, check=False) == -3        # fewer than eight 128-byte steps
    a = torch.zeros((384, 1024), dtype=torch.int8, device="cuda")
    b = torch.zeros((128, 1024), dtype=torch.int8, device="cuda")
    c = torch.zeros((384, 128), device="cuda")
    assert lib.gemm_nt(a, b, c, L.I8, L.F32, tile_config=PING, check=False) == -3        # m not a multiple of 256


@pytest.mark.parametrize("ab", ["i8", "e4m3"])
@pytest.mark.parametrize("normalize,use_rope", [(True, True), (True, False), (False, True)])
def test_row_tile_normalize_rope_epilogue_equals_the_ring_kernel(lib, ab, normalize, use_rope):
    print("case ping norm/rope epilogue", ab, normalize, use_rope, flush=True)
    from tscale2_amd import lib as L
    m, n, k = 1024, 768, 1152
    g = torch.Generator(device="cuda").manual_seed(5)
    if ab == "i8":
        a = torch.randint(-90, 90, (m, k), dtype=torch.int8, device="cuda", generator=g)
        b = torch.randint(-90, 90, (n, k), dtype=torch.int8, device="cuda", generator=g)
        t = L.I8
    else:
        a, b, t = _e4m3((m, k), g, 8.0), _e4m3((n, k), g, 8.0), L.E4M3
    a[300:310] = 0
    m_live = 900
    rope = None
    if use_rope:
        ang = torch.rand((m, 64), device="cuda", generator=g) * 6.28
        rope = torch.stack([torch.cos(ang), torch.sin(ang)], dim=2).reshape(m, 128).contiguous()
    res = []
    for cfg in (1, PING | shrink(3)):
        got = torch.full((m, n), 9, dtype=torch.int16, device="cuda")
        got_sc = torch.full((n // 128, m), -2.0, device="cuda")
        lib.gemm_nt(a, b, got, t, L.BF16, alpha=0.37, m_live=m_live, tile_config=cfg, epilogue=L.EPI_ROW_TILE_NORM, normalize=normalize,
                    vec_scale=1 / 24.0, rope=rope, tile_scale=got_sc if normalize else None)
        torch.cuda.synchronize()
        res.append((got, got_sc))
    assert torch.equal(res[0][0], res[1][0])
    if normalize:
        assert torch.equal(res[0][1][:, :m_live], res[1][1][:, :m_live])
    gf = res[1][0].view(torch.bfloat16).float()
    assert (gf[m_live:] == 0).all() and (gf[300:310] == 0).all()
