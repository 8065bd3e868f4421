"""Pins the oracle functions whose reference sources cannot be compiled without the CUDA toolkit (delta compression, per-matrix
quantiser, e4m3 device rounding rule, MoE routing, the layer glue and the head): each is checked against something the mathematics
fixes -- brute force over the code table, invariants, bilinear/adjoint identities, and finite differences of the oracle's own forward
pass, whose pieces are pinned bit-exactly against the reference build elsewhere.  A dropped term, a wrong sign or a transposed operand
in a backward function breaks the finite-difference ratio; a wrong rounding rule breaks the brute-force nearest-code check."""
import ctypes as C
import zlib

import numpy as np
import pytest

from model_harness import E4M3, I8, LT_ATT, LT_FFN, LT_MOE, Harness
from oracle_lib import Oracle, _ptr


@pytest.fixture(scope="module")
def orc():
    return Oracle()


# ---- quantisers -------------------------------------------------------------------------------------------------------------------

def test_e4m3_round_to_nearest_even_is_the_nearest_code(orc):
    """Brute force: for every probe value the chosen code is the closest finite e4m3 value; exact midpoints go to the even mantissa."""
    tab = orc.e4m3_table(hw=True).astype(np.float64)
    finite = np.array([c for c in range(256) if (c & 0x7f) != 0x7f])
    vals = tab[finite]
    r = np.random.default_rng(0)
    probes = np.concatenate([r.standard_normal(4000) * s for s in (1e-3, 0.02, 1.0, 30.0, 300.0)] + [np.array([0.0, 448.0, -448.0, 1e9, -1e9])])
    pos = np.sort(np.unique(np.abs(vals)))
    mids = (pos[1:] + pos[:-1]) / 2                                  # exact ties, representable in fp32
    probes = np.concatenate([probes, mids, -mids]).astype(np.float32)
    for x in probes:
        code = orc.lib.orc_cvt_e4m3_rne(float(x))
        got = tab[code]
        d = np.abs(vals - np.clip(float(x), -448, 448))
        best = d.min()
        assert abs(abs(got - np.clip(float(x), -448, 448)) - best) <= 1e-12, (x, code)
        if (d == best).sum() > 1 and abs(x) < 448:                   # a tie: the even code wins
            assert code % 2 == 0, (x, code)


def test_compress_delta_invariants(orc):
    """scale = maxabs/127 per (row, 128-column tile); the extreme element maps to +-127; reconstruction error <= scale/2; tile-scale
    array is [xSize/128][ySize]; an all-zero tile gets scale 0 and leaves its bytes alone."""
    r = np.random.default_rng(1)
    ys, xs = 7, 384
    data = (r.standard_normal((ys, xs)) * np.exp(r.standard_normal((ys, 1)) * 3)).astype(np.float32)
    data[2, 128:256] = 0
    delta = np.full((ys, xs), 77, np.int8)
    ts = np.zeros((xs // 128, ys), np.float32)
    orc.lib.orc_compress_delta(_ptr(data), _ptr(delta), _ptr(ts), ys, xs)
    for y in range(ys):
        for t in range(xs // 128):
            seg = data[y, t * 128:(t + 1) * 128].astype(np.float64)
            q = delta[y, t * 128:(t + 1) * 128].astype(np.float64)
            mx = np.abs(seg).max()
            if mx == 0:
                assert ts[t, y] == 0 and (q == 77).all()
                continue
            assert abs(ts[t, y] - mx / 127) <= 1.2e-7 * mx / 127
            assert np.abs(q).max() == 127 and q[np.abs(seg).argmax()] == 127 * np.sign(seg[np.abs(seg).argmax()])
            assert np.abs(q * ts[t, y] - seg).max() <= 0.5 * ts[t, y] * (1 + 1e-5)


@pytest.mark.parametrize("mode", [I8, E4M3])
def test_matrix_quantiser_is_rms_over_32(orc, mode):
    r = np.random.default_rng(2)
    w = (r.standard_normal((96, 160)) * 0.037).astype(np.float32)
    if mode == I8:
        fast = np.zeros(w.shape, np.int8)
        scale = orc.lib.orc_quantize_matrix_i8(_ptr(w), _ptr(fast), *w.shape)
        vals = fast.astype(np.float64)
        step = np.ones_like(vals)
    else:
        fast = np.zeros(w.shape, np.uint8)
        scale = orc.lib.orc_quantize_matrix_e4m3(_ptr(w), _ptr(fast), *w.shape)
        vals = orc.e4m3_table()[fast].astype(np.float64)
        step = None
    rms = np.sqrt((w.astype(np.float64) ** 2).mean())
    assert abs(scale - rms) <= 1e-6 * rms
    target = w.astype(np.float64) * 32 / rms                         # fast approximates w / (rms/32)
    if mode == I8:
        assert (np.abs(vals - target) <= 0.5 + 1e-4).all()           # nearest integer
    else:
        # the reference's CPU encoder (bit-exact against its build elsewhere) adds half an ulp, truncates and flushes values below
        # the smallest normal 2^-6 to zero: within one quantum of the target, or flushed
        quantum = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(target), 2.0 ** -6))) - 3)
        assert (np.abs(vals - target) <= np.maximum(quantum, (np.abs(target) < 2.0 ** -6) * 2.0 ** -6)).all()
    assert abs(np.sqrt((vals ** 2).mean()) - 32) < 0.2               # unit-rms matrix lands on rms 32 in code units


def test_grad_mult_is_the_power_of_two_below_128_over_max(orc):
    for mx in (1e-6, 3e-4, 0.9, 1.0, 127.9, 128.0, 5000.0):
        m = orc.lib.orc_grad_mult(mx)
        assert m == 2.0 ** np.floor(np.log2(m)), "a power of two"
        assert 64 < mx * m <= 128 + 1e-3


# ---- MoE routing ------------------------------------------------------------------------------------------------------------------

def test_moe_routing_brute_force(orc):
    r = np.random.default_rng(3)
    n, e, k = 64, 8, 3
    s = r.standard_normal((n, e)).astype(np.float32)
    s[5, 2] = s[5, 6] = s[5].max() + 1                                # a tie for the top place: the first index is taken first
    s[9, :] = 0.25                                                    # all equal: experts 0..k-1
    w = np.zeros((n, e), np.float32)
    orc.lib.orc_cpu_moe(n, e, k, _ptr(s), _ptr(w))
    for t in range(n):
        order = sorted(range(e), key=lambda i: (-s[t, i], i))[:k]     # top-k by value, ties to the lower index
        sel = np.nonzero(w[t])[0]
        assert sorted(order) == sorted(sel.tolist())
        assert abs((w[t].astype(np.float64) ** 2).sum() - e) < 1e-4
        a, b = order[0], order[-1]
        assert abs(w[t, a] / w[t, b] - np.exp((s[t, a] - s[t, b]) * 0.5)) < 1e-5 * w[t, a] / w[t, b]
    assert np.nonzero(w[9])[0].tolist() == [0, 1, 2] and np.nonzero(w[5])[0].tolist()[:1] == [2]


def test_moe_routing_backward_by_finite_differences(orc):
    r = np.random.default_rng(4)
    n, e, k = 16, 8, 2
    s = (r.standard_normal((n, e)) * 2).astype(np.float32)
    g = r.standard_normal((n, e)).astype(np.float32)

    def fwd(x):
        w = np.zeros((n, e), np.float32)
        x = np.ascontiguousarray(x, np.float32)
        orc.lib.orc_cpu_moe(n, e, k, _ptr(x), _ptr(w))
        return w.astype(np.float64)

    w = np.ascontiguousarray(fwd(s), np.float32)
    ds = g.copy()
    orc.lib.orc_cpu_backprop_moe(n, e, _ptr(w), _ptr(ds))
    assert np.abs((ds.astype(np.float64) * (w != 0)).sum(1)).max() > 0
    assert (ds[w == 0] == 0).all(), "unselected experts receive no gradient"
    eps = 1e-2
    for _ in range(6):
        d = r.standard_normal((n, e)).astype(np.float32) * (w != 0)   # move selected logits only: the selection stays fixed
        fd = ((fwd(s + eps * d) - fwd(s - eps * d)) * g).sum() / (2 * eps)
        an = (ds.astype(np.float64) * d).sum()
        assert abs(fd - an) <= 2e-3 * max(1, abs(an)), (fd, an)


def test_expert_scaling_is_bilinear_and_contract_layouts_invert(orc):
    r = np.random.default_rng(5)
    n, e, width = 5, 4, 32
    moe = r.standard_normal((n, e)).astype(np.float32)
    rg = r.standard_normal((n, width)).astype(np.float32)
    g = r.standard_normal((n, width)).astype(np.float32)
    out = rg.copy()
    orc.lib.orc_scale_experts(n, e, width, _ptr(moe), _ptr(out))
    assert np.allclose(out, rg * np.repeat(moe, width // e, axis=1), rtol=1e-6)
    grad_moe = np.zeros((n, e), np.float32)
    grad_rg = g.copy()
    orc.lib.orc_backprop_scale_experts(n, e, width, _ptr(moe), _ptr(rg), _ptr(grad_moe), _ptr(grad_rg))
    lhs = (out.astype(np.float64) * g).sum()                          # f is bilinear: <f, G> = <moe, dMoe> = <rg, dRg>
    assert abs(lhs - (moe.astype(np.float64) * grad_moe).sum()) < 1e-4 * abs(lhs) + 1e-5
    assert abs(lhs - (rg.astype(np.float64) * grad_rg).sum()) < 1e-4 * abs(lhs) + 1e-5
    xp, es, xs = 3, 4, 5
    src = np.arange(xp * es * xs, dtype=np.float32).reshape(xp * es, xs)
    res = np.zeros((es, xp * xs), np.float32)
    orc.lib.orc_fwd_contract_matrix(_ptr(src), _ptr(res), xp, es, xs)
    assert (res == src.reshape(xp, es, xs).transpose(1, 0, 2).reshape(es, xp * xs)).all()
    back = np.zeros_like(src)
    orc.lib.orc_bwd_contract_matrix(_ptr(res), _ptr(back), xp, es, xs)
    assert (back == src).all()


# ---- the layers, the head and the embedding: finite differences of the whole step ---------------------------------------------------

def _loss(h):
    return h.oracle_step(want_deltas=False)


def _fd_ratio(h, mat, delta, r, eps):
    """(<delta, D> / n_targets) / d(mean log p)/d(eps) along a direction D of one dequantised matrix.  D is half random, half the
    delta itself (both at the matrix' rms): the random half checks the delta's direction, the other half keeps the derivative well away
    from zero, so that the ratio is conditioned well enough for a tolerance of 5e-3.  The derivative is the Richardson extrapolation of
    the central differences at eps and eps / 2 (error O(eps^4)); the oracle returns the loss as a double."""
    rms = np.float32(np.sqrt((mat.deq.astype(np.float64) ** 2).mean()))
    d = r.standard_normal(mat.deq.shape).astype(np.float32) * rms * np.float32(0.5)
    drms = np.sqrt((delta.astype(np.float64) ** 2).mean())
    if drms > 0:
        d += (delta.astype(np.float64) * (0.5 * rms / drms)).astype(np.float32)
    keep = mat.deq.copy()

    def central(e):
        mat.deq[...] = keep + np.float32(e) * d
        lp = _loss(h)
        mat.deq[...] = keep - np.float32(e) * d
        lm = _loss(h)
        mat.deq[...] = keep
        return (lp - lm) / (2 * e)
    fd = (4 * central(eps / 2) - central(eps)) / 3
    an = (delta.astype(np.float64) * d).sum() / (h.target >= 0).sum()
    return an / fd, fd


def _check_ratio(h, mat, delta, expect, eps, what):
    """With experts in the model a finite step can flip a selection (a jump in the loss); the same direction is then retried with
    smaller steps and two of them have to agree with the analytic value -- a wrong gradient agrees at none."""
    steps = [eps] if h.experts == 0 else [eps / k for k in (1, 2.5, 5, 10, 25, 50, 100)]
    need = 1 if h.experts == 0 else 2
    seed = zlib.crc32(str(what).encode())
    got = []
    for e in steps:
        ratio, fd = _fd_ratio(h, mat, delta, np.random.default_rng(seed), e)
        got.append((e, ratio, fd))
    good = [g for g in got if abs(g[2]) > 1e-5 and abs(g[1] / expect - 1) < 5e-3]
    assert len(good) >= need, (what, expect, got)


@pytest.mark.parametrize("kind", ["dense", "moe"])
def test_deltas_are_the_gradient_of_the_log_likelihood(kind):
    """Every delta the backward emits equals sqrt(fan_in) * d(sum log p(target))/dW (the forward divides each product by sqrt(fan_in),
    SumRankOne does not; src/gpt/compute/cpu_util.cpp:8-67), the embedding delta equals the plain gradient.  Checked by central
    differences of the oracle's own forward pass along random directions, for every matrix of every layer type."""
    if kind == "dense":
        h = Harness(I8, 128, 1, 1, 2, 32, 2, 16, wide_window=8, seed=11, std=1.0)
    else:
        h = Harness(E4M3, 128, 1, 1, 1, 32, 2, 16, wide_window=8, experts=4, selected=2, xp=128, seed=12, std=1.0)
    # the quantised weights are what the forward multiplies with; perturb those (fp32 views), not the codes.  The step is small for
    # the MoE model: a larger one flips expert selections, where the loss is not differentiable
    eps = 2e-2 if kind == "dense" else 5e-3
    h.oracle_step()
    deltas = [[d.copy() for d in ds] for ds in h.ref_delta]
    d_embed, d_final = h.ref_delta_embed.copy(), h.ref_delta_final.copy()
    r = np.random.default_rng(7)
    seen = set()
    for layer in range(h.depth):
        lt = int(h.lt[layer])
        seen.add(lt)
        for i, m in enumerate(h.layers[layer]):
            if lt == LT_MOE and i == 2:
                fan_in = h.xp * h.experts                               # contract multiplies as [dim][experts*xp]
            else:
                fan_in = m.deq.shape[1]
            _check_ratio(h, m, deltas[layer][i], np.sqrt(fan_in), eps, (layer, lt, i))
    assert {LT_ATT, LT_FFN} <= seen if kind == "dense" else LT_MOE in seen
    _check_ratio(h, h.final, d_final, np.sqrt(h.dim), eps, "final")
    _check_ratio(h, h.embed, d_embed, 1.0, eps, "embedding")
