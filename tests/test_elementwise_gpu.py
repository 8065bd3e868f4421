"""GPU parity of the bandwidth-bound fused kernels against the CPU oracle.
fp32 results: <= 1e-5 relative (different summation order of the 128-element reductions); bf16/e4m3 outputs: one rounding step of
the output format (2^-8 / 2^-4 relative); int8 bytes: exact except on rounding boundaries."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")
from oracle_lib import Oracle, _ptr  # noqa: E402


@pytest.fixture(scope="module")
def L():
    from tscale2_amd import lib
    lib.load()
    return lib


@pytest.fixture(scope="module")
def orc():
    return Oracle()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def e4m3_decode(orc, t):
    return orc.e4m3_table(hw=True)[t.cpu().numpy().astype(np.uint8)]


def test_e4m3_conversion_matches_rne_rule(L, orc):
    """device fp32->e4m3 (used by every e4m3 store) against the round-to-nearest-even, saturating rule, over a dense sweep"""
    print("case e4m3 cvt", flush=True)
    r = np.random.default_rng(1)
    tab = orc.e4m3_table()
    pos = np.sort(np.unique(np.abs(tab[(np.arange(256) & 0x7f) != 0x7f])))
    mids = (pos[1:] + pos[:-1]) / 2
    x = np.concatenate([pos, -pos, mids, -mids, np.nextafter(mids, np.float32(1e9)), np.nextafter(mids, np.float32(0)),
                        r.standard_normal(20000) * 30, r.standard_normal(4000) * 0.01, [500, -500, 1e6, 448, 464, 1e-9]]).astype(np.float32)
    n = (x.size + 127) // 128 * 128
    x = np.concatenate([x, np.zeros(n - x.size, np.float32)]).reshape(-1, 128)
    rows = x.shape[0]
    gate = torch.full((rows, 128), 100.0, device="cuda").bfloat16()  # sigmoid(200) == 1 exactly -> res = vals
    # vals must be representable: route fp32 through scale_grad instead (gradFast = grad * 1)
    g = dev(x)
    fast = torch.zeros((rows, 128), dtype=torch.uint8, device="cuda")
    mx = torch.tensor([128.0], device="cuda")  # gradMult = 1
    gs = torch.zeros(2, device="cuda")
    L.call("ts2_scale_grad", mx, None, g, fast, L.E4M3, rows, gs[0:1], gs[1:2])
    torch.cuda.synchronize()
    assert gs.cpu().tolist() == [1.0, 1.0]
    want = np.array([orc.lib.orc_cvt_e4m3_rne(C.c_float(v)) for v in x.ravel()], np.uint8).reshape(x.shape)
    got = fast.cpu().numpy()
    bad = got != want
    # -0 vs +0 for tiny negatives is the only tolerated difference
    assert not np.any(bad & ~((got & 0x7f) == 0) | bad & ~((want & 0x7f) == 0)), (x[bad][:10], got[bad][:10], want[bad][:10])


@pytest.mark.parametrize("norm_type", ["i8", "e4m3"])
def test_layer_normalize_and_backprop(L, orc, norm_type):
    print(f"case tilenorm {norm_type}", flush=True)
    r = np.random.default_rng(2)
    len_, len_round, dim = 200, 256, 384
    state = r.standard_normal((len_round, dim)).astype(np.float32) * 3
    state[7, 128:256] = 0
    nt = L.I8 if norm_type == "i8" else L.E4M3
    tdt = torch.int8 if norm_type == "i8" else torch.uint8
    ns = torch.full((len_round, dim), 9, dtype=tdt, device="cuda")
    sc = torch.full((dim // 128, len_round), -1.0, device="cuda")
    L.call("ts2_layer_normalize_state_vecs", dev(state), L.F32, len_, len_round, 1 / 24.0, ns, nt, sc)
    torch.cuda.synchronize()
    want = orc.normalize_state(state[:len_], dim // 128)  # unit-rms tiles
    got_scale = sc.cpu().numpy()
    rms = np.sqrt((state[:len_].reshape(len_, -1, 128).astype(np.float64) ** 2).mean(-1))
    np.testing.assert_allclose(got_scale[:, :len_].T, rms / 24, rtol=1e-5)
    assert np.all(got_scale[:, len_:] == 0)
    vals = ns.cpu().numpy().astype(np.float32) if norm_type == "i8" else e4m3_decode(orc, ns)
    assert np.all(vals[len_:] == 0)
    # stored value = normalised * 24, rounded to the storage grid (i8: +-0.5; e4m3: 2^-4 relative)
    if norm_type == "i8":
        assert np.abs(vals[:len_] - np.clip(want * 24, -128, 127)).max() <= 0.5 + 1e-3
    else:
        np.testing.assert_allclose(vals[:len_], want * 24, rtol=2 ** -4, atol=2 ** -9)

    # backward, fused: dequantised source = vals * scale (what the kernel sees); oracle on exactly that source
    src = vals[:len_] * np.repeat(got_scale[:, :len_].T, 128, axis=1)
    dn = r.standard_normal((len_, dim)).astype(np.float32)
    grad0 = r.standard_normal((len_, dim)).astype(np.float32)
    comb, gscale, gmult = 0.7, 0.5, 4.0
    want_g = grad0 + orc.normalize_state_backward(src, dn * np.float32(comb * gscale), dim // 128)
    sg = dev(grad0)
    fast = torch.zeros((len_, dim), dtype=torch.bfloat16, device="cuda")
    scal = dev(np.array([comb, gscale, gmult, 0.0], np.float32))
    L.call("ts2_backprop_layer_normalize", ns, nt, sc, dev(dn), scal[0:1], scal[1:2], scal[2:3], sg, fast.view(torch.int16), L.BF16, scal[3:4], len_)
    torch.cuda.synchronize()
    np.testing.assert_allclose(sg.cpu().numpy(), want_g, rtol=1e-5, atol=2e-5)
    np.testing.assert_allclose(fast.float().cpu().numpy(), want_g * gmult, rtol=2 ** -8, atol=1e-4)
    np.testing.assert_allclose(scal[3].item(), np.abs(want_g).max(), rtol=1e-5)

    # final variant: no add, pad rows cleared, e4m3 fast gradient
    sg2 = torch.full((len_round, dim), 5.0, device="cuda")
    fast2 = torch.full((len_round, dim), 9, dtype=torch.uint8, device="cuda")
    mx = torch.zeros(1, device="cuda")
    L.call("ts2_backprop_final_normalize", len_, len_round, ns, nt, sc, dev(dn), sg2, fast2, L.E4M3, mx)
    torch.cuda.synchronize()
    want_f = orc.normalize_state_backward(src, dn, dim // 128)
    np.testing.assert_allclose(sg2.cpu().numpy()[:len_], want_f, rtol=1e-5, atol=2e-5)
    assert np.all(sg2.cpu().numpy()[len_:] == 0) and np.all(fast2.cpu().numpy()[len_:] == 0)
    np.testing.assert_allclose(e4m3_decode(orc, fast2)[:len_], want_f, rtol=2 ** -4, atol=2 ** -9)


def test_scale_grad(L, orc):
    print("case scale_grad", flush=True)
    r = np.random.default_rng(3)
    g = (r.standard_normal((130, 256)) * 1e-3).astype(np.float32)
    mx = float(np.abs(g).max())
    want_mult = orc.lib.orc_grad_mult(C.c_float(mx))
    assert want_mult == 2.0 ** np.floor(np.log2(128 / mx))
    fast = torch.zeros((130, 256), dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(2, device="cuda")
    L.call("ts2_scale_grad", dev(np.array([mx], np.float32)), None, dev(g), fast.view(torch.int16), L.BF16, 130, out[0:1], out[1:2])
    torch.cuda.synchronize()
    assert out.cpu().tolist() == [1 / want_mult, want_mult]
    np.testing.assert_allclose(fast.float().cpu().numpy(), g * want_mult, rtol=2 ** -8)
    # unchanged multiplier: fast gradient is left alone
    fast.fill_(3.0)
    L.call("ts2_scale_grad", dev(np.array([mx], np.float32)), out[1:2], dev(g), fast.view(torch.int16), L.BF16, 130, out[0:1], out[1:2])
    torch.cuda.synchronize()
    assert torch.all(fast == 3.0)


def test_lolu_forward_backward(L, orc):
    print("case lolu", flush=True)
    r = np.random.default_rng(4)
    len_, len_round, dim = 100, 128, 256
    gate = torch.from_numpy((r.standard_normal((len_, dim)) * 4).astype(np.float32)).bfloat16()
    vals = torch.from_numpy((r.standard_normal((len_, dim)) * 24).astype(np.float32)).bfloat16()
    gnp, vnp = gate.float().numpy(), vals.float().numpy()
    res = torch.full((len_round, dim), 7, dtype=torch.int8, device="cuda")
    L.call("ts2_matrix_lolu", len_, len_round, gate.cuda().view(torch.int16), vals.cuda().view(torch.int16), 1.0, res, L.I8)
    torch.cuda.synchronize()
    want = orc.lolu(gnp, vnp)
    got = res.cpu().numpy().astype(np.float32)
    assert np.abs(got[:len_] - np.clip(want, -128, 127)).max() <= 0.5 + 2e-3 and np.all(got[len_:] == 0)

    # FFN backward: vals are the normalised wide in 1/24 units, tile scale restores the un-normalised wide
    grad = r.standard_normal((len_, dim)).astype(np.float32)
    vs = 1 / 24.0
    tsc = (r.random((dim // 128, len_)) + 0.5).astype(np.float32) * np.float32(vs)
    wide_norm = vnp * np.float32(vs)
    wide = vnp * np.repeat(tsc.T, 128, axis=1)
    dgate, dvals = orc.backprop_lolu(gnp, wide_norm, grad)
    dwide = orc.normalize_state_backward(wide, dvals, dim // 128)
    gg = torch.zeros((len_round, dim), dtype=torch.bfloat16, device="cuda")
    gv = torch.zeros((len_round, dim), dtype=torch.bfloat16, device="cuda")
    L.call("ts2_backprop_row_tile_normalize_lolu", len_, len_round, gate.cuda().view(torch.int16), vals.cuda().view(torch.int16), vs, dev(tsc),
           dev(grad), L.F32, gg.view(torch.int16), gv.view(torch.int16), L.BF16)
    torch.cuda.synchronize()
    np.testing.assert_allclose(gg.float().cpu().numpy()[:len_], dgate, rtol=2 ** -7, atol=1e-5)
    np.testing.assert_allclose(gv.float().cpu().numpy()[:len_], dwide, rtol=2 ** -7, atol=2e-4)

    # attention backward: dScale fused
    ds = torch.full((dim // 128, len_round), -1.0, device="cuda")
    L.call("ts2_backprop_lolu_dscale", len_, len_round, gate.cuda().view(torch.int16), vals.cuda().view(torch.int16), vs, dev(grad), L.F32,
           gg.view(torch.int16), L.BF16, gv.view(torch.int16), L.BF16, ds)
    torch.cuda.synchronize()
    np.testing.assert_allclose(gv.float().cpu().numpy()[:len_], dvals, rtol=2 ** -7, atol=1e-5)
    want_ds = np.zeros((dim // 128, len_), np.float32)
    orc.lib.orc_compute_dscale(len_, dim // 128, 128, _ptr(wide_norm), _ptr(dvals), _ptr(want_ds))
    np.testing.assert_allclose(ds.cpu().numpy()[:, :len_], want_ds, rtol=1e-4, atol=1e-4)
    assert np.all(ds.cpu().numpy()[:, len_:] == 0)


def test_ffn_lolu_backward_and_forward_with_eight_elements_per_lane(L, orc):
    """bf16 gradient in, e4m3 gradients out (the model's fp8 FFN backward) and the e4m3 forward take the kernels with eight elements
    per lane: compared with the oracle on the same bf16 inputs, within the e4m3 rounding (2^-4 relative, half a denormal step
    absolute), pad rows zero; odd row counts and a tile count that leaves half-filled waves."""
    print("case lolu e4m3 8-wide", flush=True)
    r = np.random.default_rng(14)
    len_, len_round, dim = 301, 384, 384
    gate = torch.from_numpy((r.standard_normal((len_, dim)) * 2).astype(np.float32)).bfloat16()
    vals = torch.from_numpy((r.standard_normal((len_, dim)) * 24).astype(np.float32)).bfloat16()
    grad = torch.from_numpy((r.standard_normal((len_, dim)) * 8).astype(np.float32)).bfloat16()
    gnp, vnp, dnp = gate.float().numpy(), vals.float().numpy(), grad.float().numpy()
    vs = 1 / 24.0
    tsc = (r.random((dim // 128, len_)) + 0.5).astype(np.float32) * np.float32(vs)
    tsc[1, 7] = 0                                                     # a zero tile: zero source, zero gradient
    vnp_z = vnp.copy(); vnp_z[7, 128:256] = 0
    vals = torch.from_numpy(vnp_z).bfloat16()
    wide_norm = vnp_z * np.float32(vs)
    wide = vnp_z * np.repeat(tsc.T, 128, axis=1)
    dgate, dvals = orc.backprop_lolu(gnp, wide_norm, dnp)
    dwide = orc.normalize_state_backward(wide, dvals, dim // 128)
    gg = torch.full((len_round, dim), 9, dtype=torch.uint8, device="cuda")
    gv = torch.full((len_round, dim), 9, dtype=torch.uint8, device="cuda")
    L.call("ts2_backprop_row_tile_normalize_lolu", len_, len_round, gate.cuda().view(torch.int16), vals.cuda().view(torch.int16), vs, dev(tsc),
           grad.cuda().view(torch.int16), L.BF16, gg, gv, L.E4M3)
    torch.cuda.synchronize()
    got_g, got_v = gg.view(torch.float8_e4m3fn).float().cpu().numpy(), gv.view(torch.float8_e4m3fn).float().cpu().numpy()
    for name, got, want in (("dgate", got_g, dgate), ("dwide", got_v, dwide)):
        assert np.all(got[len_:] == 0)
        excess = np.abs(got[:len_] - np.clip(want, -448, 448)) - (np.abs(want) * 2.0 ** -4 + 2.0 ** -10 * 1.01)
        i = np.unravel_index(np.argmax(excess), excess.shape)
        assert excess[i] <= 0, (name, i, got[:len_][i], want[i])
    assert np.all(got_v[7, 128:256] == 0)
    # forward with the e4m3 result
    res = torch.full((len_round, dim), 9, dtype=torch.uint8, device="cuda")
    L.call("ts2_matrix_lolu", len_, len_round, gate.cuda().view(torch.int16), vals.cuda().view(torch.int16), 0.5, res, L.E4M3)
    torch.cuda.synchronize()
    want = orc.lolu(gnp, vnp_z) * 0.5
    got = res.view(torch.float8_e4m3fn).float().cpu().numpy()
    assert np.all(got[len_:] == 0)
    assert np.all(np.abs(got[:len_] - np.clip(want, -448, 448)) <= np.abs(want) * 2.0 ** -4 + 2.0 ** -10 * 1.01)
    # a result whose rows start 8 bytes off a 16-byte boundary takes the kernel with eight elements per lane: same bytes
    wide_res = torch.full((len_round, dim + 8), 9, dtype=torch.uint8, device="cuda")
    L.call("ts2_matrix_lolu", len_, len_round, gate.cuda().view(torch.int16), vals.cuda().view(torch.int16), 0.5, wide_res[:, 8:], L.E4M3)
    torch.cuda.synchronize()
    assert torch.equal(wide_res[:, 8:], res) and torch.all(wide_res[:, :8] == 9)


def test_ffn_lolu_backward_that_also_writes_the_transposed_gradients(L, orc):
    """ts2_backprop_row_tile_normalize_lolu_t: same bytes as ts2_backprop_row_tile_normalize_lolu for bf16 gradients and e4m3 results
    (itself checked against the oracle above), and the two transposed copies are exactly those bytes transposed, pad rows (columns of
    the copies) zero."""
    print("case lolu e4m3 with transposed copies", flush=True)
    r = np.random.default_rng(16)
    len_, len_round, dim = 301, 384, 384
    gate = torch.from_numpy((r.standard_normal((len_, dim)) * 2).astype(np.float32)).bfloat16().cuda().view(torch.int16)
    vnp = (r.standard_normal((len_, dim)) * 24).astype(np.float32)
    vnp[7, 128:256] = 0
    vals = torch.from_numpy(vnp).bfloat16().cuda().view(torch.int16)
    grad = torch.from_numpy((r.standard_normal((len_, dim)) * 8).astype(np.float32)).bfloat16().cuda().view(torch.int16)
    vs = 1 / 24.0
    tsc = (r.random((dim // 128, len_)) + 0.5).astype(np.float32) * np.float32(vs)
    tsc[1, 7] = 0
    gg = torch.full((len_round, dim), 9, dtype=torch.uint8, device="cuda")
    gv = torch.full((len_round, dim), 9, dtype=torch.uint8, device="cuda")
    L.call("ts2_backprop_row_tile_normalize_lolu", len_, len_round, gate, vals, vs, dev(tsc), grad, L.BF16, gg, gv, L.E4M3)
    gg2, gv2 = torch.full_like(gg, 5), torch.full_like(gv, 5)
    ggT = torch.full((dim, len_round), 5, dtype=torch.uint8, device="cuda")
    gvT = torch.full((dim, len_round), 5, dtype=torch.uint8, device="cuda")
    L.call("ts2_backprop_row_tile_normalize_lolu_t", len_, len_round, gate, vals, vs, dev(tsc), grad, gg2, gv2, ggT, gvT)
    torch.cuda.synchronize()
    assert torch.equal(gg2, gg) and torch.equal(gv2, gv)
    assert torch.equal(ggT, gg.T.contiguous()) and torch.equal(gvT, gv.T.contiguous())
    assert torch.all(gg2[len_:] == 0) and torch.all(gvT[:, len_:] == 0)


def test_attention_lolu_backward_with_eight_elements_per_lane(L, orc):
    """bf16 gradient in, e4m3 gate gradient and bf16 value gradient out (the model's fp8 attention backward) takes the kernel with
    eight elements per lane: gate gradient within the e4m3 rounding of the oracle's, value gradient within the bf16 rounding, the
    per-(head, row) sums <values, value gradient> within fp32 summation error, pad rows zero."""
    print("case attention lolu 8-wide", flush=True)
    r = np.random.default_rng(15)
    len_, len_round, dim = 301, 384, 384
    gate = torch.from_numpy((r.standard_normal((len_, dim)) * 2).astype(np.float32)).bfloat16()
    vals = torch.from_numpy((r.standard_normal((len_, dim)) * 24).astype(np.float32)).bfloat16()
    grad = torch.from_numpy((r.standard_normal((len_, dim)) * 8).astype(np.float32)).bfloat16()
    gnp, vnp, dnp = gate.float().numpy(), vals.float().numpy(), grad.float().numpy()
    vs = 1 / 24.0
    vals_scaled = vnp * np.float32(vs)
    dgate, dvals = orc.backprop_lolu(gnp, vals_scaled, dnp)
    want_ds = np.zeros((dim // 128, len_), np.float32)
    orc.lib.orc_compute_dscale(len_, dim // 128, 128, _ptr(vals_scaled), _ptr(dvals), _ptr(want_ds))
    gg = torch.full((len_round, dim), 9, dtype=torch.uint8, device="cuda")
    gv = torch.full((len_round, dim), 9, dtype=torch.bfloat16, device="cuda")
    ds = torch.full((dim // 128, len_round), -1.0, device="cuda")
    L.call("ts2_backprop_lolu_dscale", len_, len_round, gate.cuda().view(torch.int16), vals.cuda().view(torch.int16), vs,
           grad.cuda().view(torch.int16), L.BF16, gg, L.E4M3, gv.view(torch.int16), L.BF16, ds)
    torch.cuda.synchronize()
    got_g = gg.view(torch.float8_e4m3fn).float().cpu().numpy()
    got_v = gv.float().cpu().numpy()
    assert np.all(got_g[len_:] == 0) and np.all(got_v[len_:] == 0)
    assert np.all(np.abs(got_g[:len_] - np.clip(dgate, -448, 448)) <= np.abs(dgate) * 2.0 ** -4 + 2.0 ** -10 * 1.01)
    np.testing.assert_allclose(got_v[:len_], dvals, rtol=2 ** -7, atol=1e-5)
    np.testing.assert_allclose(ds.cpu().numpy()[:, :len_], want_ds, rtol=1e-4, atol=2e-4)
    assert np.all(ds.cpu().numpy()[:, len_:] == 0)


def test_row_max_quantise(L, orc):
    print("case rowmax", flush=True)
    r = np.random.default_rng(5)
    len_, len_round, dim = 300, 384, 1280
    x = (r.standard_normal((len_, dim)) * r.random((len_, 1)) * 5).astype(np.float32)
    x[11] = 0
    want = np.zeros((len_, dim), np.int8); wscale = np.zeros(len_, np.float32)
    orc.lib.orc_quant_rowmax_i8(_ptr(x), _ptr(want), _ptr(wscale), len_, dim)
    dst = torch.full((len_round, dim), 3, dtype=torch.int8, device="cuda")
    rs = torch.full((len_round,), -1.0, device="cuda")
    L.call("ts2_normalize_vecs_row_max", len_, len_round, dev(x), L.F32, None, dst, rs)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(rs.cpu().numpy()[:len_], wscale)
    assert np.all(rs.cpu().numpy()[len_:] == 0) and np.all(dst.cpu().numpy()[len_:] == 0)
    np.testing.assert_array_equal(dst.cpu().numpy()[:len_], want)


@pytest.mark.parametrize("dim,col_scale", [(512, False), (1536, True), (4096, True)])
def test_row_max_quantise_of_bf16_rows_by_one_wave_per_row(L, orc, dim, col_scale):
    """bf16 rows whose length is a multiple of 512 (up to 4096) take the wave-per-row kernel: bytes, row scales and row maxima must
    equal the oracle's on the same bf16 values, with and without column scales; pad rows are cleared."""
    print("case rowmax bf16 wave", dim, col_scale, flush=True)
    r = np.random.default_rng(dim)
    len_, len_round = 9000, 9216                       # more rows than waves in the launch: with column scales a wave walks several rows
    x16 = torch.from_numpy((r.standard_normal((len_, dim)) * r.random((len_, 1)) * 5).astype(np.float32)).bfloat16()
    x16[11] = 0
    cs = (r.random(dim) + 0.5).astype(np.float32) if col_scale else None
    x = x16.float().numpy()
    xs = x * cs[None, :] if col_scale else x
    want = np.zeros((len_, dim), np.int8); wscale = np.zeros(len_, np.float32)
    orc.lib.orc_quant_rowmax_i8(_ptr(np.ascontiguousarray(xs)), _ptr(want), _ptr(wscale), len_, dim)
    dst = torch.full((len_round, dim), 3, dtype=torch.int8, device="cuda")
    rs = torch.full((len_round,), -1.0, device="cuda")
    rmax = torch.full((len_round,), -1.0, device="cuda")
    L.call("ts2_normalize_vecs_row_max2", len_, len_round, x16.cuda().view(torch.int16), L.BF16, dev(cs) if col_scale else None, dst, rs, rmax)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(rs.cpu().numpy()[:len_], wscale)
    np.testing.assert_array_equal(dst.cpu().numpy()[:len_], want)
    np.testing.assert_array_equal(rmax.cpu().numpy()[:len_], np.abs(x).max(1))
    assert np.all(rs.cpu().numpy()[len_:] == 0) and np.all(dst.cpu().numpy()[len_:] == 0) and np.all(rmax.cpu().numpy()[len_:] == 0)


def test_transpose_and_ktile_quant(L, orc):
    print("case transpose", flush=True)
    r = np.random.default_rng(6)
    len_, len_round, dim, kt = 700, 768, 256, 256
    b = r.integers(-128, 128, (len_, dim), dtype=np.int8)
    dst = torch.full((dim, len_round), 5, dtype=torch.int8, device="cuda")
    L.call("ts2_transpose_quant", len_, len_round, dev(b), L.I8, None, None, 0, None, dst, L.I8, None)
    torch.cuda.synchronize()
    got = dst.cpu().numpy()
    np.testing.assert_array_equal(got[:, :len_], b.T)
    assert np.all(got[:, len_:] == 0)
    # gather variant
    idx = r.integers(-1, len_, len_round).astype(np.int32)
    L.call("ts2_transpose_quant", len_round, len_round, dev(b), L.I8, None, None, 0, dev(idx), dst, L.I8, None)
    torch.cuda.synchronize()
    want = np.where(idx[None, :] >= 0, b[np.maximum(idx, 0)].T, 0)
    np.testing.assert_array_equal(dst.cpu().numpy(), want)

    # k-tile quantisation from fp32 with a per-row multiplier
    x = (r.standard_normal((len_, dim)) * (1 + 10 * r.random((len_, 1)))).astype(np.float32)
    rm = (r.random(len_) + 0.5).astype(np.float32)
    xs = x * rm[:, None]
    want_q = np.zeros((len_, dim), np.int8); want_s = np.zeros(len_round // kt, np.float32)
    orc.lib.orc_quant_ktile_i8(_ptr(xs), _ptr(want_q), _ptr(want_s), len_, dim, kt)
    tmax = torch.full((len_round // kt,), 7.0, device="cuda")
    L.call("ts2_tile_absmax", len_, dev(x), L.F32, dev(rm), kt, tmax, 1)
    tsc = torch.zeros(len_round // kt, device="cuda")
    L.call("ts2_transpose_quant", len_, len_round, dev(x), L.F32, dev(rm), tmax, kt, None, dst, L.I8, tsc)
    torch.cuda.synchronize()
    np.testing.assert_allclose(tsc.cpu().numpy(), want_s, rtol=3e-7)
    got = dst.cpu().numpy()[:, :len_].T.astype(np.int32)
    np.testing.assert_array_equal(got, want_q)


@pytest.mark.parametrize("src,dim", [("bf16", 1536), ("bf16", 4096), ("f32", 1280), ("bf16", 640)])
def test_row_max_quantise_with_dither_equals_the_oracle_given_the_same_noise(L, orc, src, dim):
    """ts2_normalize_vecs_row_max_dither: the reference rounds x / scale + u, u uniform in (-0.5, 0.5) (src/gpt/compute/row_scale.cuh:32-35).
    The library's u is a counter-based hash of (seed, row, column); the oracle takes the same values as an array: bytes and scales must
    agree bit for bit on the wave-per-row kernel (bf16, dim a multiple of 512) and on the workgroup-per-row kernel alike."""
    from test_oracle_own_contract import dither_noise
    print("case rowmax dither", src, dim, flush=True)
    r = np.random.default_rng(dim)
    len_, len_round, seed = 1000, 1024, 0x1234567
    x = (r.standard_normal((len_, dim)) * r.random((len_, 1)) * 5).astype(np.float32)
    x[11] = 0
    if src == "bf16":
        x16 = torch.from_numpy(x).bfloat16()
        x = x16.float().numpy()
        dsrc, ty = x16.cuda().view(torch.int16), L.BF16
    else:
        dsrc, ty = dev(x), L.F32
    noise = dither_noise(seed, len_, dim)
    want = np.zeros((len_, dim), np.int8); wscale = np.zeros(len_, np.float32)
    orc.lib.orc_quant_rowmax_i8_noise(_ptr(np.ascontiguousarray(x)), _ptr(noise), _ptr(want), _ptr(wscale), len_, dim)
    dst = torch.full((len_round, dim), 3, dtype=torch.int8, device="cuda")
    rs = torch.full((len_round,), -1.0, device="cuda")
    L.call("ts2_normalize_vecs_row_max_dither", len_, len_round, dsrc, ty, None, dst, rs, None, seed)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(rs.cpu().numpy()[:len_], wscale)
    np.testing.assert_array_equal(dst.cpu().numpy()[:len_], want)
    assert np.all(dst.cpu().numpy()[len_:] == 0)
    plain = np.zeros((len_, dim), np.int8)
    orc.lib.orc_quant_rowmax_i8(_ptr(np.ascontiguousarray(x)), _ptr(plain), _ptr(wscale), len_, dim)
    assert 0.2 < (plain != want).mean() < 0.6                                   # the dither does move a good part of the bytes
    # seed 0 is the deterministic quantiser
    L.call("ts2_normalize_vecs_row_max_dither", len_, len_round, dsrc, ty, None, dst, rs, None, 0)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(dst.cpu().numpy()[:len_], plain)


def test_dithered_quantiser_is_unbiased_on_the_device(L):
    """E[q * scale] = x: rows of one constant (plus one extreme element that fixes the scale at 1) quantised under the dither average to
    the constant; rounding to nearest gives the nearest integer instead."""
    print("case rowmax dither unbiased", flush=True)
    len_, dim = 4096, 512
    for c in (0.3, -1.45, 17.02):
        x = torch.full((len_, dim), c, device="cuda")
        x[:, 0] = 127
        dst = torch.zeros((len_, dim), dtype=torch.int8, device="cuda")
        rs = torch.zeros(len_, device="cuda")
        L.call("ts2_normalize_vecs_row_max_dither", len_, len_, x, L.F32, None, dst, rs, None, 4242)
        torch.cuda.synchronize()
        assert bool((rs == 1).all())
        mean = dst[:, 1:].double().mean().item()
        assert abs(mean - c) < 2e-3, (c, mean)
        L.call("ts2_normalize_vecs_row_max_dither", len_, len_, x, L.F32, None, dst, rs, None, 0)
        torch.cuda.synchronize()
        assert dst[:, 1:].double().mean().item() == round(c)


def test_transpose_and_ktile_quant_with_dither(L, orc):
    from test_oracle_own_contract import dither_noise
    print("case transpose dither", flush=True)
    r = np.random.default_rng(16)
    len_, len_round, dim, kt, seed = 700, 768, 256, 256, 99991
    x16 = torch.from_numpy((r.standard_normal((len_, dim)) * (1 + 10 * r.random((len_, 1)))).astype(np.float32)).bfloat16()
    x = x16.float().numpy()
    rm = (r.random(len_) + 0.5).astype(np.float32)
    xs = x * rm[:, None]
    noise = dither_noise(seed, len_, dim)
    want_q = np.zeros((len_, dim), np.int8); want_s = np.zeros(len_round // kt, np.float32)
    orc.lib.orc_quant_ktile_i8_noise(_ptr(xs), _ptr(noise), _ptr(want_q), _ptr(want_s), len_, dim, kt)
    tmax = torch.full((len_round // kt,), 7.0, device="cuda")
    L.call("ts2_tile_absmax", len_, x16.cuda().view(torch.int16), L.BF16, dev(rm), kt, tmax, 1)
    tsc = torch.zeros(len_round // kt, device="cuda")
    dst = torch.full((dim, len_round), 5, dtype=torch.int8, device="cuda")
    L.call("ts2_transpose_quant_dither", len_, len_round, x16.cuda().view(torch.int16), L.BF16, dev(rm), tmax, kt, None, dst, L.I8, tsc, seed)
    torch.cuda.synchronize()
    np.testing.assert_allclose(tsc.cpu().numpy(), want_s, rtol=3e-7)
    np.testing.assert_array_equal(dst.cpu().numpy()[:, :len_].T, want_q)
    assert np.all(dst.cpu().numpy()[:, len_:] == 0)
