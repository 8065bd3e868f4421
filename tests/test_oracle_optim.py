"""Pins the oracle's optimiser step (oracle/optim.c: UnpackDelta and THostModelMatrix::AddDelta restated; their reference files need
cuda_runtime.h and cannot be compiled here) by what the update rule fixes in closed form - none of these retypes the loop:
  * unpack o compress is the identity within half a quantisation step;
  * without moving average or decay a step moves every row by exactly rate * sqrt(sparsity) in rms, along its delta;
  * repeated identical deltas: the moving average and the dispersion estimate follow their geometric series;
  * weight decay alone shrinks the weights by (1 - step * l2) per step;
  * one dispersion estimate per block of rows = the mean square over the block;
  * an all-zero delta leaves the weights where they are (and produces no NaN)."""
import ctypes as C

import numpy as np
import pytest

from oracle_lib import Oracle, _ptr


class Step(C.Structure):
    _fields_ = [(n, C.c_float) for n in ("rate", "l2Reg", "beta1", "weight0", "weight1", "dispDecay")]


@pytest.fixture(scope="module")
def orc():
    o = Oracle()
    o.lib.orc_apply_delta.restype = C.c_double
    return o


def apply(orc, w, ag, delta, row_disp, sum_weight, sparsity, st):
    ys, xs = w.shape
    sw = np.array([sum_weight], np.float32)
    rs = np.zeros(ys, np.float32)
    s2 = orc.lib.orc_apply_delta(_ptr(w), _ptr(ag), _ptr(delta), ys, xs, row_disp.size, _ptr(row_disp), _ptr(sw), C.c_float(sparsity), C.byref(st), _ptr(rs))
    return s2, float(sw[0]), rs


def test_unpack_inverts_compress_within_half_a_step(orc):
    r = np.random.default_rng(41)
    ys, xs = 9, 384
    data = (r.standard_normal((ys, xs)) * np.exp(r.standard_normal((ys, 1)) * 2)).astype(np.float32)
    data[4, 128:256] = 0
    q = np.zeros((ys, xs), np.int8); ts = np.zeros((xs // 128, ys), np.float32)
    orc.lib.orc_compress_delta(_ptr(data), _ptr(q), _ptr(ts), ys, xs)
    back = np.full((ys, xs), 7, np.float32)
    orc.lib.orc_unpack_delta(_ptr(q), _ptr(ts), _ptr(back), ys, xs, 0)
    step = np.repeat(ts.T, 128, axis=1)
    assert (np.abs(back - data) <= step * 0.5 * (1 + 1e-6)).all()
    assert (back[4, 128:256] == 0).all()
    twice = back.copy()
    orc.lib.orc_unpack_delta(_ptr(q), _ptr(ts), _ptr(twice), ys, xs, 1)       # add = 1 accumulates
    np.testing.assert_array_equal(twice, back + back)


def test_plain_step_has_unit_length_per_row(orc):
    r = np.random.default_rng(42)
    ys, xs = 6, 256
    w0 = r.standard_normal((ys, xs)).astype(np.float32)
    delta = (r.standard_normal((ys, xs)) * np.exp(r.standard_normal((ys, 1)) * 3)).astype(np.float32)  # rows of very different size
    w = w0.copy(); ag = np.zeros_like(w); rd = np.zeros(ys, np.float32)
    st = Step(0.01, 0, 0, 1, 0, 0)       # DisableMovingAverage
    s2, sw, rs = apply(orc, w, ag, delta, rd, 0.0, 0.25, st)
    move = w - w0
    step = 0.01 * np.sqrt(0.25)
    np.testing.assert_allclose(np.sqrt((move.astype(np.float64) ** 2).mean(1)), step, rtol=1e-5)   # every row moves by the step, whatever its size
    cos = (move * delta).sum(1) / np.sqrt((move.astype(np.float64) ** 2).sum(1) * (delta.astype(np.float64) ** 2).sum(1))
    np.testing.assert_allclose(cos, 1, rtol=1e-6)                                                  # ... along its delta
    np.testing.assert_allclose(s2, (w.astype(np.float64) ** 2).sum(), rtol=1e-6)
    assert sw == 1.0
    np.testing.assert_allclose(rs, 1 / np.sqrt((delta.astype(np.float64) ** 2).mean(1)), rtol=1e-5)


def test_moving_average_and_dispersion_follow_their_geometric_series(orc):
    r = np.random.default_rng(43)
    ys, xs, n = 4, 128, 5
    delta = r.standard_normal((ys, xs)).astype(np.float32)
    w = np.zeros((ys, xs), np.float32); ag = np.zeros_like(w); rd = np.zeros(ys, np.float32)
    beta1, decay = 0.9, 0.8
    st = Step(0.0, 0, beta1, 1, 0, decay)   # rate 0: only the statistics move
    sw = 0.0
    for _ in range(n):
        _, sw, rs = apply(orc, w, ag, delta, rd, sw, 1.0, st)
    geo = (1 - decay ** n) / (1 - decay)
    np.testing.assert_allclose(sw, geo, rtol=1e-6)
    ms = (delta.astype(np.float64) ** 2).mean(1)
    np.testing.assert_allclose(rd, ms * geo, rtol=1e-5)                       # rowDisp = mean square * (1 + d + d^2 + ...)
    np.testing.assert_allclose(rs, 1 / np.sqrt(ms), rtol=1e-5)                # normalised by sumWeight: the scale is stationary
    d_norm = delta / np.sqrt(ms)[:, None]
    np.testing.assert_allclose(ag, d_norm * (1 - beta1 ** n), rtol=2e-5, atol=1e-6)   # (1-b) * sum b^k = 1 - b^n
    assert (w == 0).all()


def test_weight_decay_and_zero_delta(orc):
    r = np.random.default_rng(44)
    ys, xs = 3, 128
    w0 = r.standard_normal((ys, xs)).astype(np.float32)
    w = w0.copy(); ag = np.zeros_like(w); rd = np.zeros(ys, np.float32)
    st = Step(0.02, 0.5, 0, 1, 0, 0.9)
    s2, sw, rs = apply(orc, w, ag, np.zeros_like(w), rd, 0.0, 4.0, st)
    step = 0.02 * np.sqrt(4.0)
    np.testing.assert_allclose(w, w0 * np.float32(1 - step * 0.5), rtol=1e-6)
    assert np.isfinite(w).all() and (rs == 0).all() and (ag == 0).all()


def test_block_dispersion_is_the_mean_over_the_block(orc):
    r = np.random.default_rng(45)
    ys, xs = 8, 128
    delta = (r.standard_normal((ys, xs)) * np.arange(1, ys + 1)[:, None]).astype(np.float32)
    w = np.zeros((ys, xs), np.float32); ag = np.zeros_like(w); rd = np.zeros(2, np.float32)   # two blocks of four rows
    st = Step(1.0, 0, 0, 1, 0, 0)
    _, _, rs = apply(orc, w, ag, delta, rd, 0.0, 1.0, st)
    ms = (delta.astype(np.float64) ** 2).reshape(2, 4 * xs).mean(1)
    np.testing.assert_allclose(rd, ms, rtol=1e-5)
    np.testing.assert_allclose(rs, np.repeat(1 / np.sqrt(ms), 4), rtol=1e-5)
    np.testing.assert_allclose(w, delta * np.repeat(1 / np.sqrt(ms), 4)[:, None].astype(np.float32), rtol=1e-5)  # the block moves by rms 1 as a whole
