"""Linear-layer backward (dX = dY*W, delta = dY^T*X) on the GPU against the oracle's fp32 CPU path (MulBackwardWithAccum,
SumRankOne).  The GPU path quantises dY to int8 (per row for dX, per k-tile for the delta) or takes e4m3 operands, so agreement is
bounded by the quantisation step: max |err| <= 1e-2 * max |ref| (the stated tolerance for 8-bit gradients); int32 partial sums are
checked bit-exactly in test_gemm_gpu.py."""
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


def make_case(orc, seed, len_, src_dim, grad_dim, fp8):
    r = np.random.default_rng(seed)
    w = (r.standard_normal((grad_dim, src_dim)) * 0.02).astype(np.float32)
    if fp8:
        fast = np.zeros((grad_dim, src_dim), np.uint8)
        sko = orc.lib.orc_quantize_matrix_e4m3(_ptr(w), _ptr(fast), grad_dim, src_dim)
        wq = orc.e4m3_table()[fast] * np.float32(sko / 32)
    else:
        fast = np.zeros((grad_dim, src_dim), np.int8)
        sko = orc.lib.orc_quantize_matrix_i8(_ptr(w), _ptr(fast), grad_dim, src_dim)
        wq = fast.astype(np.float32) * np.float32(sko / 32)
    # layer input: unit-rms tiles stored as 8-bit in 1/24 units (the reference's NormState format)
    x = orc.normalize_state(r.standard_normal((len_, src_dim)).astype(np.float32), src_dim // 128)
    dy = (r.standard_normal((len_, grad_dim)) * (0.2 + r.random((len_, 1)))).astype(np.float32)
    return w, fast, float(sko), wq, x, dy


@pytest.mark.parametrize("len_,src_dim,grad_dim", [(500, 256, 384), (1024, 512, 256)])
def test_int8_linear_backward(L, orc, len_, src_dim, grad_dim):
    print(f"case linear i8 {len_} {src_dim} {grad_dim}", flush=True)
    len_round = (len_ + 511) // 512 * 512
    w, fast, sko, wq, x, dy = make_case(orc, 11, len_, src_dim, grad_dim, False)
    x8 = orc.convert_i8(x, 24.0)
    xq = x8.astype(np.float32) / 24
    # oracle on exactly the operands the device sees (dequantised weights and inputs, bf16 gradient)
    dy16 = torch.from_numpy(dy).bfloat16()
    dyf = dy16.float().numpy()
    ref_dx = orc.mul_backward_accum(np.zeros((len_, src_dim), np.float32), wq, dyf)
    ref_delta = orc.sum_rank_one(xq, dyf)

    bufs = L.MatMulBuffers(L.I8, len_round, src_dim, grad_dim, k_tile=256)
    x8d = torch.zeros((len_round, src_dim), dtype=torch.int8, device="cuda")
    x8d[:len_] = torch.from_numpy(x8).cuda()
    dyd = dy16.cuda()
    wscale = torch.tensor([sko], device="cuda")
    dx = torch.full((len_round, src_dim), 9.0, device="cuda")
    bufs.backprop_multi(len_, torch.from_numpy(fast).cuda(), dyd.view(torch.int16), L.BF16)
    bufs.backprop(len_, None, (1 / 32) / np.sqrt(src_dim), wscale, dx, L.F32)
    bufs.backprop_delta(len_, x8d, None, dyd.view(torch.int16), L.BF16)
    torch.cuda.synchronize()
    got_dx = dx.cpu().numpy()
    assert np.all(got_dx[len_:] == 0)

    # (1) same contract on the CPU: identical quantisation, exact int32 sums -> agreement to the last bit of the int8 operands and
    #     an fp32 epilogue that may differ by rounding order only
    q8 = np.zeros((len_, grad_dim), np.int8); rsc = np.zeros(len_, np.float32)
    orc.lib.orc_quant_rowmax_i8(_ptr(dyf), _ptr(q8), _ptr(rsc), len_, grad_dim)
    np.testing.assert_array_equal(bufs.t["grad8"].cpu().numpy()[:len_], q8)
    np.testing.assert_array_equal(bufs.t["grad8RowScale"].cpu().numpy()[:len_], rsc)
    np.testing.assert_array_equal(bufs.t["transformT"].cpu().numpy(), fast.T)
    same_dx = np.zeros((len_, src_dim), np.float32)
    import ctypes as C
    orc.lib.orc_gemm_i8_nt_rowscale(_ptr(q8), _ptr(rsc), _ptr(np.ascontiguousarray(fast.T)), C.c_float(np.float32((1 / 32) / np.sqrt(src_dim)) * np.float32(sko)),
                                    _ptr(same_dx), len_, src_dim, grad_dim, 0)
    np.testing.assert_allclose(got_dx[:len_], same_dx, rtol=2e-6, atol=1e-9)
    kt = 256
    qk = np.zeros((len_round, grad_dim), np.int8); tsc = np.zeros(len_round // kt, np.float32)
    dypad = np.zeros((len_round, grad_dim), np.float32); dypad[:len_] = dyf
    orc.lib.orc_quant_ktile_i8(_ptr(dypad), _ptr(qk), _ptr(tsc), len_round, grad_dim, kt)
    np.testing.assert_array_equal(bufs.t["gradT"].cpu().numpy(), qk.T)
    x8pad = np.zeros((len_round, src_dim), np.int8); x8pad[:len_] = x8
    np.testing.assert_array_equal(bufs.t["srcT"].cpu().numpy(), x8pad.T)
    acc = np.zeros((grad_dim, src_dim), np.float32)
    orc.lib.orc_gemm_i8_nt_ktile(_ptr(np.ascontiguousarray(qk.T)), _ptr(np.ascontiguousarray(x8pad.T)), _ptr(tsc), kt, C.c_float(1.0), _ptr(acc),
                                 grad_dim, src_dim, len_round)
    want_delta = np.zeros((grad_dim, src_dim), np.int8); want_ts = np.zeros((src_dim // 128, grad_dim), np.float32)
    orc.lib.orc_compress_delta(_ptr(acc), _ptr(want_delta), _ptr(want_ts), grad_dim, src_dim)
    np.testing.assert_allclose(bufs.delta_tile_scale.cpu().numpy(), want_ts, rtol=2e-6)
    dd = np.abs(bufs.delta.cpu().numpy().astype(np.int32) - want_delta)
    assert dd.max() <= 1 and (dd != 0).mean() < 1e-3

    # (2) against the reference's fp32 CPU path: bounded by the int8 quantisation step of dY (per row: 1/254 of the row maximum per
    #     element for dX; per k-tile for the delta, plus 1/254 of the row-tile maximum for the packed output)
    def errs(got, ref):
        d = got - ref
        return np.sqrt((d ** 2).mean()) / np.sqrt((ref ** 2).mean()), np.abs(d).max() / np.abs(ref).max()
    rms, mx = errs(got_dx[:len_], ref_dx)
    print("dX rel err rms/max", rms, mx)
    assert rms <= 1e-2 and mx <= 3e-2
    got_delta = bufs.delta_fp32().cpu().numpy() / 24  # X was stored in 1/24 units
    rms, mx = errs(got_delta, ref_delta)
    print("delta rel err rms/max", rms, mx)
    assert rms <= 2e-2 and mx <= 3e-2
    # adding a second source accumulates
    bufs.backprop(len_, None, (1 / 32) / np.sqrt(src_dim), wscale, dx, L.F32, add=True)
    torch.cuda.synchronize()
    np.testing.assert_allclose(dx.cpu().numpy(), 2 * got_dx, rtol=1e-6)


def test_fp8_linear_backward(L, orc):
    print("case linear fp8", flush=True)
    len_, src_dim, grad_dim = 900, 256, 512
    len_round = 1024
    w, fast, sko, wq, x, dy = make_case(orc, 12, len_, src_dim, grad_dim, True)
    tab = orc.e4m3_table(hw=True)
    xe = np.array([orc.lib.orc_cvt_e4m3_rne(__import__("ctypes").c_float(v)) for v in (x * 24).ravel()], np.uint8).reshape(x.shape)
    xq = tab[xe] / 24
    # fast gradient: fp32 gradient times the power-of-two multiplier, stored as e4m3
    mult = orc.lib.orc_grad_mult(__import__("ctypes").c_float(float(np.abs(dy).max())))
    dye = np.array([orc.lib.orc_cvt_e4m3_rne(__import__("ctypes").c_float(v)) for v in (dy * mult).ravel()], np.uint8).reshape(dy.shape)
    dyq = tab[dye] / np.float32(mult)
    ref_dx = orc.mul_backward_accum(np.zeros((len_, src_dim), np.float32), wq, dyq)
    ref_delta = orc.sum_rank_one(xq, dyq)

    bufs = L.MatMulBuffers(L.E4M3, len_round, src_dim, grad_dim)
    xd = torch.zeros((len_round, src_dim), dtype=torch.uint8, device="cuda"); xd[:len_] = torch.from_numpy(xe).cuda()
    dyd = torch.zeros((len_round, grad_dim), dtype=torch.uint8, device="cuda"); dyd[:len_] = torch.from_numpy(dye).cuda()
    gscale = torch.tensor([1 / mult], device="cuda")
    dx = torch.zeros((len_round, src_dim), device="cuda")
    bufs.backprop_multi(len_, torch.from_numpy(fast).cuda(), None, L.E4M3)
    bufs.backprop(len_, dyd, (1 / 32) / np.sqrt(src_dim) * sko, gscale, dx, L.F32)
    bufs.backprop_delta(len_, xd, None, dyd, L.E4M3, gscale)
    torch.cuda.synchronize()
    # operands are identical on both sides; only fp32 accumulation differs -> 1e-4 (MFMA fp8 adder-tree precision)
    err = np.abs(dx.cpu().numpy()[:len_] - ref_dx).max() / np.abs(ref_dx).max()
    print("fp8 dX rel err", err)
    assert err <= 1e-4
    # the packed delta adds its own int8 rounding: 1/254 of each row-tile maximum
    got_delta = bufs.delta_fp32().cpu().numpy() / 24
    err = np.abs(got_delta - ref_delta).max() / np.abs(ref_delta).max()
    print("fp8 delta rel err", err)
    assert err <= 5e-3
    # the caller's word that the pad rows hold zeros (they do: xd, dyd above): the delta product reads both arrays as they lie,
    # transposes nothing (the transpose scratch keeps its marker bytes) and gives the same bytes and tile scales
    rows = L.MatMulBuffers(L.E4M3, len_round, src_dim, grad_dim)
    rows.c.padRowsZero = 1
    rows.t["gradT"].fill_(0x5A); rows.t["srcT"].fill_(0x5A)
    rows.delta.fill_(77); rows.delta_tile_scale.fill_(-1)
    rows.backprop_delta(len_, xd, None, dyd, L.E4M3, gscale)
    torch.cuda.synchronize()
    assert torch.equal(rows.delta, bufs.delta) and torch.equal(rows.delta_tile_scale, bufs.delta_tile_scale)
    assert (rows.t["gradT"] == 0x5A).all() and (rows.t["srcT"] == 0x5A).all()
    assert not (bufs.t["gradT"] == 0x5A).all()            # the transposing sequence did write its scratch
    # whole 128-row groups: the same without the flag
    full = L.MatMulBuffers(L.E4M3, len_round, src_dim, grad_dim)
    full.t["gradT"].fill_(0x5A)
    full.backprop_delta(len_round, xd, None, dyd, L.E4M3, gscale)
    torch.cuda.synchronize()
    assert torch.equal(full.delta, bufs.delta) and torch.equal(full.delta_tile_scale, bufs.delta_tile_scale)
    assert (full.t["gradT"] == 0x5A).all()


@pytest.mark.parametrize("dims", [(256, 512), (384, 128)])
@pytest.mark.parametrize("mode", ["i8", "e4m3"])
def test_delta_as_stored_slices_plus_pack_matches_the_single_pass(L, orc, mode, dims):
    """BackpropDelta with a `partial` workspace: the token axis is cut into slices whose products are stored in fp32 and packed from
    their sum.  Same quantised operands and the same exact int32 sums per k-tile; only the association of the fp32 additions differs
    (per slice, then across slices), so packed bytes may differ from the single-pass result by one unit in rare places."""
    print("case delta split slices", mode, dims, flush=True)
    (src_dim, grad_dim), len_, kt, splits = dims, 2048, 256, 4   # (384, 128): 128x128 tiles, as for the select matrix of a MoE layer
    r = np.random.default_rng(21)
    dy = (r.standard_normal((len_, grad_dim)) * (0.2 + r.random((len_, 1)))).astype(np.float32)
    x = orc.normalize_state(r.standard_normal((len_, src_dim)).astype(np.float32), src_dim // 128)
    if mode == "i8":
        m = L.I8
        xs = torch.from_numpy(orc.convert_i8(x, 24.0)).cuda()
        g = torch.from_numpy(dy).bfloat16().cuda().view(torch.int16)
        gt = L.BF16
    else:
        m = L.E4M3
        xs = (torch.from_numpy(x).cuda() * 24).to(torch.float8_e4m3fn).view(torch.uint8)
        g = (torch.from_numpy(dy).cuda() * 64).to(torch.float8_e4m3fn).view(torch.uint8)
        gt = L.E4M3
    one = L.MatMulBuffers(m, len_, src_dim, grad_dim, k_tile=kt)
    cut = L.MatMulBuffers(m, len_, src_dim, grad_dim, k_tile=kt, splits=splits)
    cut.delta.fill_(55)
    one.backprop_delta(len_, xs, None, g, gt, alpha=0.5)
    cut.backprop_delta(len_, xs, None, g, gt, alpha=0.5)
    torch.cuda.synchronize()
    a, b = one.delta_fp32().cpu().numpy(), cut.delta_fp32().cpu().numpy()
    np.testing.assert_allclose(cut.delta_tile_scale.cpu().numpy(), one.delta_tile_scale.cpu().numpy(), rtol=3e-6)
    dd = np.abs(cut.delta.cpu().numpy().astype(np.int32) - one.delta.cpu().numpy())
    assert dd.max() <= 1 and (dd != 0).mean() < 2e-3
    assert np.abs(a - b).max() <= np.abs(a).max() / 127 * 1.01
    if mode == "i8":
        # the slices themselves: partial i equals the k-tile sum over its own token range (exact int32 per k-tile; the fp32 additions
        # of the tiles are fused multiply-adds on the device, separate operations in the oracle)
        part = cut.t["partial"].cpu().numpy().reshape(splits, grad_dim, src_dim)
        qk = cut.t["gradT"].cpu().numpy().T.copy(); x8 = cut.t["srcT"].cpu().numpy().T.copy(); tsc = cut.t["tileScale"].cpu().numpy()
        import ctypes as C
        per = len_ // splits
        for i in range(splits):
            acc = np.zeros((grad_dim, src_dim), np.float32)
            orc.lib.orc_gemm_i8_nt_ktile(_ptr(np.ascontiguousarray(qk[i * per:(i + 1) * per].T)), _ptr(np.ascontiguousarray(x8[i * per:(i + 1) * per].T)),
                                         _ptr(np.ascontiguousarray(tsc[i * per // kt:(i + 1) * per // kt])), kt, C.c_float(1.0), _ptr(acc), grad_dim, src_dim, per)
            assert np.abs(part[i] - acc).max() <= 2e-7 * np.abs(acc).max() * (per // kt)


def test_delta_from_shared_row_maxima_is_identical(L, orc):
    """BackpropMulti can leave the abs-max of every gradient row behind; BackpropDelta then builds its k-tile scales from those instead
    of reading the gradient again.  Same maxima, same scales: the packed delta is identical."""
    print("case shared row maxima", flush=True)
    len_, len_round, src_dim, grad_dim, kt = 900, 1024, 256, 384, 256
    r = np.random.default_rng(31)
    dy = torch.from_numpy((r.standard_normal((len_, grad_dim)) * (0.2 + r.random((len_, 1)))).astype(np.float32)).bfloat16().cuda().view(torch.int16)
    x8 = torch.zeros((len_round, src_dim), dtype=torch.int8, device="cuda")
    x8[:len_] = torch.from_numpy(orc.convert_i8(orc.normalize_state(r.standard_normal((len_, src_dim)).astype(np.float32), 2), 24.0)).cuda()
    w8 = torch.randint(-100, 100, (grad_dim, src_dim), dtype=torch.int8, device="cuda")
    col = torch.rand(grad_dim, device="cuda") + 0.5
    xs = torch.rand(len_round, device="cuda") + 0.5
    res = []
    for share in (False, True):
        b = L.MatMulBuffers(L.I8, len_round, src_dim, grad_dim, k_tile=kt, share_row_max=share)
        b.backprop_multi(len_, w8, dy, L.BF16, col)
        b.backprop_delta(len_, x8, xs, dy, L.BF16)
        torch.cuda.synchronize()
        res.append((b.delta.cpu().numpy(), b.delta_tile_scale.cpu().numpy(), b.t["tileScale"].cpu().numpy()))
    for a, c in zip(*res):
        np.testing.assert_array_equal(a, c)


@pytest.mark.parametrize("mode", ["e4m3", "i8"])
def test_grouped_backprop_equals_the_products_added_one_after_the_other(L, orc, mode):
    """ts2_matmul_backprop_group over four matrices that share their input against four Backprop() calls (store, then accumulate).
    fp8 on the 256 grid runs as one launch (same fp32 MFMA sums, rescaled between products, one rounding of the total: a few ulps of
    the largest partial sum); int8 falls back to the sequence itself and must be identical."""
    print("case grouped dX", mode, flush=True)
    from tscale2_amd import lib as LL
    len_, src_dim, grad_dim, n = 700, 512, 256, 4
    len_round = 768
    r = np.random.default_rng(31)
    m = L.E4M3 if mode == "e4m3" else L.I8
    bufs, grads, scales = [], [], []
    for i in range(n):
        w = (r.standard_normal((grad_dim, src_dim)) * 20).astype(np.float32)
        dy = (r.standard_normal((len_round, grad_dim)) * (0.3 + r.random((len_round, 1)))).astype(np.float32)
        dy[len_:] = 0
        if mode == "e4m3":
            wf = (torch.from_numpy(w).cuda()).to(torch.float8_e4m3fn).view(torch.uint8)
            g = (torch.from_numpy(dy).cuda() * 16).to(torch.float8_e4m3fn).view(torch.uint8)
            gt = L.E4M3
        else:
            wf = torch.from_numpy(np.clip(np.rint(w), -127, 127).astype(np.int8)).cuda()
            g = torch.from_numpy(dy).bfloat16().cuda().view(torch.int16)
            gt = L.BF16
        b = L.MatMulBuffers(m, len_round, src_dim, grad_dim)
        b.backprop_multi(len_, wf, g, gt)
        bufs.append(b); grads.append(g)
        scales.append(None if i == 3 else torch.full((1,), 0.6 + 0.3 * i, device="cuda"))
    alphas = [0.01 * (i + 1) for i in range(n)]
    c0 = torch.randn((len_round, src_dim), device="cuda")
    for add in (False, True):
        want = c0.clone()
        for i in range(n):
            bufs[i].backprop(len_, grads[i] if mode == "e4m3" else None, alphas[i], scales[i], want, L.F32, add=add or i > 0)
        got = c0.clone()
        LL.matmul_backprop_group(bufs, len_, grads if mode == "e4m3" else [None] * n, alphas, scales, got, L.F32, add=add)
        torch.cuda.synchronize()
        if mode == "i8":
            assert torch.equal(got, want)
        else:
            scale = want[:len_].abs().max().item()
            assert (got[:len_] - want[:len_]).abs().max().item() <= 4e-6 * scale


def test_transposes_left_by_the_caller_are_used_as_they_are(L, orc):
    """transformTValid: BackpropMulti does not transpose the matrix again, so the product uses whatever transformT holds (here the
    transpose of the first matrix although another one is passed); gradTValid: BackpropDelta contracts over the gradT it is given (here
    the transposed gradient placed there by the caller, while the gradient argument holds other values).  With the flags cleared the
    arguments count again."""
    print("case caller-provided transposes", flush=True)
    len_, src_dim, grad_dim = 512, 256, 384
    g = torch.Generator(device="cuda").manual_seed(5)
    f8 = lambda r, c, s: (torch.randn((r, c), device="cuda", generator=g) * s).to(torch.float8_e4m3fn).view(torch.uint8)
    w1, w2 = f8(grad_dim, src_dim, 8), f8(grad_dim, src_dim, 8)
    grad, other = f8(len_, grad_dim, 16), f8(len_, grad_dim, 16)
    x = f8(len_, src_dim, 8)
    b = L.MatMulBuffers(L.E4M3, len_, src_dim, grad_dim)

    def dx(w):
        out = torch.zeros((len_, src_dim), device="cuda")
        b.backprop_multi(len_, w, grad, L.E4M3)
        b.backprop(len_, grad, 0.01, None, out, L.F32)
        torch.cuda.synchronize()
        return out
    first, second = dx(w1), dx(w2)
    assert not torch.equal(first, second)
    b.c.transformTValid = 1                       # transformT holds w2^T
    assert torch.equal(dx(w1), second)
    b.c.transformTValid = 0
    assert torch.equal(dx(w1), first)

    def delta(gr):
        b.backprop_delta(len_, x, None, gr, L.E4M3, alpha=0.5)
        torch.cuda.synchronize()
        return b.delta.clone(), b.delta_tile_scale.clone()
    d1, s1 = delta(grad)
    d2, s2 = delta(other)
    assert not torch.equal(d1, d2)
    b.t["gradT"].copy_(grad.T)                    # the producer's transposed copy
    b.c.gradTValid = 1
    d3, s3 = delta(other)
    assert torch.equal(d3, d1) and torch.equal(s3, s1)
    b.c.gradTValid = 0
    d4, s4 = delta(other)
    assert torch.equal(d4, d2) and torch.equal(s4, s2)


# ---- rows sorted by scale before the delta product (the reference's order) -----------------------------------------------------------

def _sort_dev(L, key, mult=None):
    n = key.size
    order = torch.full((n,), -1, dtype=torch.int32, device="cuda"); tmp = torch.empty_like(order)
    L.call("ts2_sort_rows_by_scale", n, torch.from_numpy(key).cuda(), None if mult is None else torch.from_numpy(mult).cuda(), order, tmp)
    torch.cuda.synchronize()
    return order.cpu().numpy()


def test_row_sort_reproduces_the_reference_order(L, orc):
    """ts2_sort_rows_by_scale on the input of the reference's own sort test: the hash of the order it holds (cuda_sort.cu:247), and the
    oracle's order on other lengths and with a row multiplier"""
    import ctypes as C
    import os
    print("case row sort", flush=True)
    orc.lib.orc_sort_result_hash.restype = C.c_uint32
    x = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_golden.npz"))["sort.mt1313_real3"]
    got = _sort_dev(L, x)
    assert orc.lib.orc_sort_result_hash(_ptr(np.ascontiguousarray(got)), x.size) == 1749808112
    r = np.random.default_rng(31)
    for n in (1, 2, 63, 499, 500, 700, 5000, 32768, 70001):
        key = np.exp(r.standard_normal(n) * 3).astype(np.float32)
        key[r.random(n) < 0.05] = 0                                            # zero rows sort first
        if n > 40:
            key[30:40] = key[7]                                                # equal keys: ascending rows below 500, descending from 500 on
        mult = (r.standard_normal(n) * 2).astype(np.float32) if n % 2 else None  # the key is |mult| * max
        eff = key if mult is None else (key * np.abs(mult)).astype(np.float32)
        want = np.zeros(n, np.int32)
        orc.lib.orc_hist_sort_stable(_ptr(eff), n, _ptr(want), 0)           # fewer than 500: the exact sort, as in the reference
        np.testing.assert_array_equal(_sort_dev(L, key, mult), want)


@pytest.mark.parametrize("k_tile", [128, 512])
def test_int8_delta_with_sorted_rows_same_contract(L, orc, k_tile):
    """BackpropDelta with sortRows: the same contract on the CPU (the oracle's sort, rows gathered in that order, k-tile quantiser, exact
    int32 sums per k-tile, packed delta) gives the same bytes; the row order and both transposed operands are checked on the way"""
    import ctypes as C
    print("case int8 delta, sorted rows", k_tile, flush=True)
    len_, src_dim, grad_dim = 1500, 256, 384
    len_round = (len_ + 511) // 512 * 512
    r = np.random.default_rng(32)
    x = orc.normalize_state(r.standard_normal((len_, src_dim)).astype(np.float32), src_dim // 128)
    x8 = orc.convert_i8(x, 24.0)
    dy16 = torch.from_numpy((r.standard_normal((len_, grad_dim)) * np.exp(r.standard_normal((len_, 1)) * 2)).astype(np.float32)).bfloat16()
    dyf = dy16.float().numpy()
    w8 = r.integers(-127, 128, (grad_dim, src_dim), dtype=np.int8)
    bufs = L.MatMulBuffers(L.I8, len_round, src_dim, grad_dim, k_tile=k_tile, share_row_max=True, sort_rows=True)
    x8d = torch.zeros((len_round, src_dim), dtype=torch.int8, device="cuda"); x8d[:len_] = torch.from_numpy(x8).cuda()
    dyd = dy16.cuda().view(torch.int16)
    bufs.backprop_multi(len_, torch.from_numpy(w8).cuda(), dyd, L.BF16)   # leaves the row maxima the sort keys come from
    bufs.backprop_delta(len_, x8d, None, dyd, L.BF16)
    torch.cuda.synchronize()
    key = np.abs(dyf).max(1).astype(np.float32)
    order = np.zeros(len_, np.int32)
    orc.lib.orc_hist_sort_stable(_ptr(key), len_, _ptr(order), 1)
    np.testing.assert_array_equal(bufs.t["rowOrder"].cpu().numpy()[:len_], order)
    dys = np.zeros((len_round, grad_dim), np.float32); dys[:len_] = dyf[order]
    xs = np.zeros((len_round, src_dim), np.int8); xs[:len_] = x8[order]
    qk = np.zeros((len_round, grad_dim), np.int8); tsc = np.zeros(len_round // k_tile, np.float32)
    orc.lib.orc_quant_ktile_i8(_ptr(dys), _ptr(qk), _ptr(tsc), len_round, grad_dim, k_tile)
    np.testing.assert_array_equal(bufs.t["gradT"].cpu().numpy(), qk.T)
    np.testing.assert_array_equal(bufs.t["srcT"].cpu().numpy(), xs.T)
    acc = np.zeros((grad_dim, src_dim), np.float32)
    orc.lib.orc_gemm_i8_nt_ktile(_ptr(np.ascontiguousarray(qk.T)), _ptr(np.ascontiguousarray(xs.T)), _ptr(tsc), k_tile, C.c_float(1.0), _ptr(acc),
                                 grad_dim, src_dim, len_round)
    want = np.zeros((grad_dim, src_dim), np.int8); want_ts = np.zeros((src_dim // 128, grad_dim), np.float32)
    orc.lib.orc_compress_delta(_ptr(acc), _ptr(want), _ptr(want_ts), grad_dim, src_dim)
    np.testing.assert_allclose(bufs.delta_tile_scale.cpu().numpy(), want_ts, rtol=2e-6)
    dd = np.abs(bufs.delta.cpu().numpy().astype(np.int32) - want)
    assert dd.max() <= 1 and (dd != 0).mean() < 1e-3


def test_int8_delta_precision_on_heavy_tailed_rows(L, orc):
    """What the common scale of a k-tile costs when the gradient rows differ in magnitude (log-normal row scales, sigma 0.5 and 3),
    with consecutive rows and with rows sorted by scale, against the fp32 SumRankOne of the CPU path.  int8 with one scale per k-tile
    keeps about two per cent of the delta's rms whatever the order; sorting helps where the spread is mild."""
    print("case int8 delta, heavy-tailed rows", flush=True)
    len_, src_dim, grad_dim = 4096, 256, 256
    r = np.random.default_rng(33)
    x8 = orc.convert_i8(orc.normalize_state(r.standard_normal((len_, src_dim)).astype(np.float32), src_dim // 128), 24.0)
    x8d = torch.from_numpy(x8).cuda()
    w8 = torch.from_numpy(r.integers(-127, 128, (grad_dim, src_dim), dtype=np.int8)).cuda()
    res = {}
    for sigma in (0.5, 3.0):
        dy16 = torch.from_numpy((r.standard_normal((len_, grad_dim)) * np.exp(r.standard_normal((len_, 1)) * sigma)).astype(np.float32)).bfloat16()
        ref = orc.sum_rank_one(x8.astype(np.float32), dy16.float().numpy())
        for sort_rows in (False, True):
            for kt in (128, 512):
                bufs = L.MatMulBuffers(L.I8, len_, src_dim, grad_dim, k_tile=kt, share_row_max=True, sort_rows=sort_rows)
                dyd = dy16.cuda().view(torch.int16)
                bufs.backprop_multi(len_, w8, dyd, L.BF16)
                bufs.backprop_delta(len_, x8d, None, dyd, L.BF16)
                torch.cuda.synchronize()
                d = bufs.delta_fp32().cpu().numpy() - ref
                res[(sigma, sort_rows, kt)] = (float(np.sqrt((d ** 2).mean()) / np.sqrt((ref ** 2).mean())), float(np.abs(d).max() / np.abs(ref).max()))
                print(f"sigma {sigma} sorted {sort_rows} kTile {kt}: rms {res[(sigma, sort_rows, kt)][0]:.4f} max/max {res[(sigma, sort_rows, kt)][1]:.4f}")
    for k, (rms, mx) in res.items():
        assert rms <= 0.10 and mx <= 0.08, (k, rms, mx)
    # mild spread: rows of like scale share a tile once sorted, and the result is clearly closer
    assert res[(0.5, True, 128)][0] <= 0.7 * res[(0.5, False, 128)][0]
    assert res[(0.5, True, 512)][0] <= 0.8 * res[(0.5, False, 512)][0]
