"""Pins the oracle functions that state this library's own 8-bit contracts (row-max and k-tile quantisers, int8 products with row or
k-tile scales) and its small helpers, against what the mathematics fixes and against library routines: numpy's round-half-even and
int64 products, torch's bfloat16 conversion, scipy's softmax.  None of these has a counterpart the reference's CPU sources could pin."""
import ctypes as C

import numpy as np
import pytest

from oracle_lib import Oracle, _ptr


@pytest.fixture(scope="module")
def orc():
    return Oracle()


def heavy_rows(r, rows, cols):
    """rows whose magnitudes spread over orders of magnitude, one all-zero row, exact .5 ties after scaling"""
    x = (r.standard_normal((rows, cols)) * np.exp(r.standard_normal((rows, 1)) * 2.5)).astype(np.float32)
    x[3] = 0
    x[5, :8] = np.array([127, -127, 63.5, -63.5, 0.5, -0.5, 1.5, 2.5], np.float32)  # max 127 -> scale 1: the ties stay ties
    x[5, 8:] = np.clip(x[5, 8:], -100, 100)
    return x


def test_row_max_quantiser_closed_form(orc):
    """scale = maxabs(row)/127 in fp32, q = saturate(round-half-even(x * (1/scale))), zero rows give scale 0 and zero bytes"""
    r = np.random.default_rng(11)
    x = heavy_rows(r, 23, 384)
    q = np.full(x.shape, 99, np.int8); sc = np.full(x.shape[0], -1, np.float32)
    orc.lib.orc_quant_rowmax_i8(_ptr(x), _ptr(q), _ptr(sc), *x.shape)
    mx = np.abs(x).max(1)
    want_sc = (mx / np.float32(127)).astype(np.float32)
    assert np.array_equal(sc, want_sc)
    mult = np.where(mx > 0, np.float32(1) / np.where(mx > 0, want_sc, 1), 0).astype(np.float32)
    want_q = np.clip(np.rint((x * mult[:, None]).astype(np.float32)), -128, 127).astype(np.int8)
    assert np.array_equal(q, want_q)
    assert (q[3] == 0).all() and sc[3] == 0
    assert list(q[5, :8]) == [127, -127, 64, -64, 0, 0, 2, 2]            # halves go to the even neighbour
    live = mx > 0
    assert (np.abs(q[live]).max(1) == 127).all()                        # the extreme element of a row maps to +-127
    assert (np.abs(q * sc[:, None] - x) <= sc[:, None] * 0.5 * (1 + 1e-6)).all()  # error at most half a step


@pytest.mark.parametrize("k_tile,rows", [(4, 23), (8, 16), (32, 23)])
def test_k_tile_quantiser_closed_form(orc, k_tile, rows):
    """every kTile consecutive rows share scale = maxabs(tile)/127 (1 for an all-zero tile; a ragged last tile takes what is left)"""
    r = np.random.default_rng(12)
    x = heavy_rows(r, rows, 128)
    if k_tile == 4:
        x[8:12] = 0
    n_tiles = (rows + k_tile - 1) // k_tile
    q = np.full(x.shape, 99, np.int8); sc = np.full(n_tiles, -1, np.float32)
    orc.lib.orc_quant_ktile_i8(_ptr(x), _ptr(q), _ptr(sc), rows, 128, k_tile)
    for t in range(n_tiles):
        blk = x[t * k_tile:(t + 1) * k_tile]
        mx = np.abs(blk).max()
        s = np.float32(mx) / np.float32(127) if mx > 0 else np.float32(1)
        assert sc[t] == s
        want = np.clip(np.rint((blk * (np.float32(1) / s)).astype(np.float32)), -128, 127).astype(np.int8)
        assert np.array_equal(q[t * k_tile:(t + 1) * k_tile], want)
        if mx > 0:
            assert np.abs(want).max() == 127
    if k_tile == 4:
        assert sc[2] == 1 and (q[8:12] == 0).all()


def test_int8_products_against_int64(orc):
    """raw int32 sums, the row-scaled and the k-tile-scaled epilogues against an int64 numpy product: exact where the contract says
    exact (int32 sums; one rounding per fp32 multiply), saturating inputs included"""
    r = np.random.default_rng(13)
    m, n, k, kt = 9, 7, 96, 32
    a = r.integers(-128, 128, (m, k), dtype=np.int8); b = r.integers(-128, 128, (n, k), dtype=np.int8)
    a[0] = -128; b[0] = -128                                             # the largest sum a tile can hold
    ref = a.astype(np.int64) @ b.astype(np.int64).T
    c = np.zeros((m, n), np.int32)
    orc.lib.orc_gemm_i8_nt(_ptr(a), _ptr(b), _ptr(c), m, n, k)
    assert np.array_equal(c.astype(np.int64), ref) and c[0, 0] == 128 * 128 * k
    rs = (r.random(m) + 0.5).astype(np.float32)
    out = np.zeros((m, n), np.float32)
    orc.lib.orc_gemm_i8_nt_rowscale(_ptr(a), _ptr(rs), _ptr(b), C.c_float(0.37), _ptr(out), m, n, k, 0)
    want = (ref.astype(np.float32) * rs[:, None]).astype(np.float32) * np.float32(0.37)
    assert np.array_equal(out, want)
    base = out.copy()
    orc.lib.orc_gemm_i8_nt_rowscale(_ptr(a), _ptr(rs), _ptr(b), C.c_float(0.37), _ptr(out), m, n, k, 1)   # add = 1 accumulates
    assert np.array_equal(out, base + want)
    orc.lib.orc_gemm_i8_nt_rowscale(_ptr(a), None, _ptr(b), C.c_float(1.0), _ptr(out), m, n, k, 0)          # no row scale = 1
    assert np.array_equal(out, ref.astype(np.float32))
    ks = (r.random(k // kt) + 0.5).astype(np.float32)
    orc.lib.orc_gemm_i8_nt_ktile(_ptr(a), _ptr(b), _ptr(ks), kt, C.c_float(0.25), _ptr(out), m, n, k)
    acc = np.zeros((m, n), np.float32)
    for t in range(k // kt):                                             # tiles in order, fp32 adds
        part = a[:, t * kt:(t + 1) * kt].astype(np.int64) @ b[:, t * kt:(t + 1) * kt].astype(np.int64).T
        acc = (acc + ks[t] * part.astype(np.float32)).astype(np.float32)
    assert np.array_equal(out, acc * np.float32(0.25))
    # exact identity when every tile scale is the same power of two: the k-tile product is the plain product
    ks2 = np.full(k // kt, 0.5, np.float32)
    orc.lib.orc_gemm_i8_nt_ktile(_ptr(a), _ptr(b), _ptr(ks2), kt, C.c_float(1.0), _ptr(out), m, n, k)
    assert np.array_equal(out, ref.astype(np.float32) * 0.5)


def test_fp32_yardstick_product_against_float64(orc):
    r = np.random.default_rng(14)
    a = r.standard_normal((5, 40)).astype(np.float32); b = r.standard_normal((6, 40)).astype(np.float32)
    out = np.ones((5, 6), np.float32)
    orc.lib.orc_gemm_f32_nt(_ptr(a), _ptr(b), _ptr(out), 5, 6, 40, C.c_float(0.5), 1)
    want = (1 + (a.astype(np.float64) @ b.astype(np.float64).T * 0.5).astype(np.float32)).astype(np.float32)
    np.testing.assert_allclose(out, want, rtol=1e-7, atol=0)


def test_dequantisers_invert_the_code_tables(orc):
    tab = orc.e4m3_table()
    codes = np.arange(256, dtype=np.uint8)
    w = np.zeros(256, np.float32)
    orc.lib.orc_dequant_e4m3(_ptr(codes), _ptr(w), 256, C.c_float(0.75))
    assert np.array_equal(w, tab * np.float32(0.75))
    i8 = np.arange(-128, 128, dtype=np.int8)
    orc.lib.orc_dequant_i8(_ptr(i8), _ptr(w), 256, C.c_float(0.75))
    assert np.array_equal(w, i8.astype(np.float32) * np.float32(0.75))


def test_bf16_rounding_is_the_library_conversion(orc):
    torch = pytest.importorskip("torch")
    r = np.random.default_rng(15)
    x = np.concatenate([r.standard_normal(5000) * 10.0 ** r.integers(-20, 20, 5000), [0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.4e38, -3.4e38]])
    x = x.astype(np.float32)
    # exact ties: a bf16 value plus half a bf16 ulp
    b = torch.from_numpy(x).bfloat16().float().numpy()
    ties = (b.view(np.uint32) | 0x8000).view(np.float32)
    x = np.concatenate([x, ties[np.isfinite(ties)]])
    got = np.array([orc.lib.orc_bf16_round(float(v)) for v in x], np.float32)
    want = torch.from_numpy(x).bfloat16().float().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_softmax_base_two_with_the_zero_sink_in_the_maximum(orc):
    """p = 2^(logit + bias - m) / sum with m = max(0, max logit): the same as scipy's softmax of ln2 * (logit + bias); the running
    maximum starting at 0 changes nothing but the range of the exponents (src/gpt/compute/cpu_transformer.cpp:12-37)"""
    from scipy.special import softmax
    r = np.random.default_rng(16)
    logits = (r.standard_normal((6, 50)) * 4).astype(np.float32)
    logits[2] -= 30                                                     # every logit below 0: the maximum stays 0
    bias = r.standard_normal(50).astype(np.float32)
    pred = np.zeros_like(logits)
    orc.lib.orc_softmax2(_ptr(logits), _ptr(bias), _ptr(pred), 6, 50)
    want = softmax((logits.astype(np.float64) + bias) * np.log(2.0), axis=1)
    np.testing.assert_allclose(pred, want, rtol=2e-6, atol=1e-30)
    np.testing.assert_allclose(pred.sum(1), 1, rtol=1e-6)


def test_embedding_is_a_signed_gather_and_its_backward_the_scatter(orc):
    r = np.random.default_rng(17)
    n, dim, label_count = 7, 128, 12
    per = r.integers(0, 4, n)
    label_ptr = np.concatenate([[0], np.cumsum(per)]).astype(np.int32)
    ids = r.integers(0, label_count, label_ptr[-1]).astype(np.uint32)
    neg = r.random(label_ptr[-1]) < 0.4
    labels = (ids | (neg.astype(np.uint32) << 31)).astype(np.uint32)
    embed = r.standard_normal((label_count, dim)).astype(np.float32)
    state = np.full((n, dim), 5, np.float32)
    orc.lib.orc_embedding_forward(n, dim, _ptr(label_ptr), _ptr(labels), _ptr(embed), _ptr(state))
    want = np.zeros((n, dim), np.float64)
    for t in range(n):
        for k in range(label_ptr[t], label_ptr[t + 1]):
            want[t] += embed[ids[k]] * (-1 if neg[k] else 1)
    np.testing.assert_allclose(state, want, rtol=1e-6, atol=1e-6)
    grad = r.standard_normal((n, dim)).astype(np.float32)
    delta = np.zeros((label_count, dim), np.float32)
    orc.lib.orc_embedding_backward(n, dim, label_count, _ptr(label_ptr), _ptr(labels), _ptr(grad), _ptr(delta))
    # adjoint identity: <grad, forward(E)> = <delta, E> for every E
    np.testing.assert_allclose((grad.astype(np.float64) * want).sum(), (delta.astype(np.float64) * embed).sum(), rtol=1e-5)
    wd = np.zeros((label_count, dim), np.float64)
    for t in range(n):
        for k in range(label_ptr[t], label_ptr[t + 1]):
            wd[ids[k]] += grad[t] * (-1 if neg[k] else 1)
    np.testing.assert_allclose(delta, wd, rtol=1e-6, atol=1e-6)


def test_hist_sort_reproduces_the_hash_of_the_reference_sort_test(orc):
    """TestCudaSort (src/lib/cuda/cuda_sort.cu:232-250) sorts 16384 draws of TMersenne(1313).GenRandReal3() and checks the hash of the
    node ids against 1749808112: the restated order (bins of the top 13 bits ascending, descending id inside a bin) must give it"""
    import os
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_golden.npz"))
    x = gold["sort.mt1313_real3"]
    # the same stream from numpy's Mersenne twister (init_genrand(1313), (u32 + 0.5) / 2^32): the fixture is what the reference draws
    u = np.random.RandomState(1313).randint(0, 2 ** 32, x.size, dtype=np.uint64)
    assert np.array_equal(((u.astype(np.float64) + 0.5) / 4294967296.0).astype(np.float32), x)
    order = np.zeros(x.size, np.int32)
    orc.lib.orc_hist_sort_stable(_ptr(x), x.size, _ptr(order), 0)
    orc.lib.orc_sort_result_hash.restype = C.c_uint32
    assert orc.lib.orc_sort_result_hash(_ptr(order), x.size) == 1749808112
    assert sorted(order.tolist()) == list(range(x.size))
    keys = x.view(np.uint32) >> 18
    assert (np.diff(keys[order].astype(np.int64)) >= 0).all()
    same = keys[order][1:] == keys[order][:-1]
    assert (np.diff(order)[same] < 0).all()                              # descending id inside a bin
    # below 500 values the reference sorts exactly, by (score, id)
    y = np.round(x[:300] * 20) / 20
    o2 = np.zeros(300, np.int32)
    orc.lib.orc_hist_sort_stable(_ptr(y), 300, _ptr(o2), 0)
    assert np.array_equal(o2, np.lexsort((np.arange(300), y)))


def dither_noise(seed, rows, cols, row0=0):
    """the library's dither stream (include/ts2_abi.h, ts2_normalize_vecs_row_max_dither): noise[t][x] = (byte (x % 4) of
    lowbias32(seed ^ t * 0x9E3779B1 ^ (x / 4) * 0x85EBCA6B) - 127.5) / 256, in uint32 arithmetic"""
    t = (np.arange(rows, dtype=np.uint64) + row0)[:, None]
    c4 = (np.arange(cols, dtype=np.uint64) // 4)[None, :]
    m = np.uint64(0xffffffff)
    h = (np.uint64(seed) ^ ((t * np.uint64(0x9E3779B1)) & m) ^ ((c4 * np.uint64(0x85EBCA6B)) & m)) & m
    h ^= h >> np.uint64(16)
    h = (h * np.uint64(0x7FEB352D)) & m
    h ^= h >> np.uint64(15)
    h = (h * np.uint64(0x846CA68B)) & m
    h ^= h >> np.uint64(16)
    byte = (h >> (np.uint64(8) * (np.arange(cols, dtype=np.uint64) % np.uint64(4))[None, :])) & np.uint64(255)
    return ((byte.astype(np.float32) - np.float32(127.5)) * np.float32(1 / 256)).astype(np.float32)


def test_dithered_quantisers_closed_form_and_unbiased(orc):
    """q = saturate(round-half-even(fma(x, 1/scale, noise))): equal to the plain quantiser for zero noise, equal to numpy's float64
    evaluation rounded once (a fused multiply-add), and unbiased: the mean of q * scale over a uniform noise stream is x.
    The hash stream itself is uniform over its 256 levels and independent between neighbouring columns and rows."""
    r = np.random.default_rng(31)
    x = heavy_rows(r, 23, 384)
    q0 = np.zeros(x.shape, np.int8); s0 = np.zeros(23, np.float32)
    orc.lib.orc_quant_rowmax_i8(_ptr(x), _ptr(q0), _ptr(s0), *x.shape)
    zero = np.zeros_like(x)
    q = np.full(x.shape, 99, np.int8); sc = np.full(23, -1, np.float32)
    orc.lib.orc_quant_rowmax_i8_noise(_ptr(x), _ptr(zero), _ptr(q), _ptr(sc), *x.shape)
    assert np.array_equal(q, q0) and np.array_equal(sc, s0)
    noise = dither_noise(12345, *x.shape)
    assert noise.min() >= -0.5 + 1 / 512 - 1e-7 and noise.max() <= 0.5 - 1 / 512 + 1e-7
    orc.lib.orc_quant_rowmax_i8_noise(_ptr(x), _ptr(noise), _ptr(q), _ptr(sc), *x.shape)
    mult = np.where(s0 > 0, np.float32(1) / np.where(s0 > 0, s0, 1), 0).astype(np.float32)
    fused = (x.astype(np.float64) * mult[:, None].astype(np.float64) + noise.astype(np.float64)).astype(np.float32)   # one rounding
    assert np.array_equal(q, np.clip(np.rint(fused), -128, 127).astype(np.int8))
    assert np.array_equal(sc, s0)
    # the stream: every level equally likely, no correlation between neighbours
    big = dither_noise(777, 512, 2048)
    levels = np.rint((big + 0.5) * 256 - 0.5).astype(np.int64)
    counts = np.bincount(levels.ravel(), minlength=256)
    assert counts.min() > 0.9 * big.size / 256 and counts.max() < 1.1 * big.size / 256
    assert abs(big.mean()) < 1e-3
    assert abs((big[:, 1:] * big[:, :-1]).mean()) < 2e-4 and abs((big[1:] * big[:-1]).mean()) < 2e-4
    # unbiased: a constant row (plus one extreme element that fixes the scale at 1) under many noise rows
    const = np.full((4096, 256), 0.3, np.float32)
    const[:, 0] = 127
    nz = dither_noise(99, *const.shape)
    qc = np.zeros(const.shape, np.int8); scc = np.zeros(4096, np.float32)
    orc.lib.orc_quant_rowmax_i8_noise(_ptr(const), _ptr(nz), _ptr(qc), _ptr(scc), *const.shape)
    assert (scc == 1).all()
    assert abs(qc[:, 1:].astype(np.float64).mean() - 0.3) < 2e-3               # round-to-nearest alone gives 0
    # k-tile form: the same noise rule with one scale per tile
    xk = heavy_rows(r, 16, 128)
    nk = dither_noise(5, 16, 128)
    qk = np.zeros(xk.shape, np.int8); sk = np.zeros(2, np.float32)
    orc.lib.orc_quant_ktile_i8_noise(_ptr(xk), _ptr(nk), _ptr(qk), _ptr(sk), 16, 128, 8)
    for t in range(2):
        blk = xk[t * 8:(t + 1) * 8]
        mx = np.abs(blk).max()
        s = np.float32(mx) / np.float32(127) if mx > 0 else np.float32(1)
        assert sk[t] == s
        f = (blk.astype(np.float64) * np.float64(np.float32(1) / s) + nk[t * 8:(t + 1) * 8].astype(np.float64)).astype(np.float32)
        assert np.array_equal(qk[t * 8:(t + 1) * 8], np.clip(np.rint(f), -128, 127).astype(np.int8))
