"""Optimiser apply on the device against the oracle (oracle/optim.c: UnpackDelta and THostModelMatrix::AddDelta restated) and, for the
requantised fast weights, against the oracle's per-matrix quantiser (quant.h:42-79) applied to the updated weights.  Every kernel of
src/gpt/matrix/agpu_cuda.cu:9-134 / agpu_cuda.cuh:35-101 is called on its own and through ts2_opt_add_delta, in both orders the
operator supports (one delta applied at once from the packed bytes; deltas accumulated in fp32, then applied)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")
from oracle_lib import Oracle, _ptr  # noqa: E402


class Step(C.Structure):
    _fields_ = [(n, C.c_float) for n in ("rate", "l2Reg", "beta1", "weight0", "weight1", "dispDecay")]


class Mat(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("strideBytes", C.c_int64), ("x", C.c_int32), ("y", C.c_int32)]


class OptMatrix(C.Structure):
    _fields_ = [("xSize", C.c_int32), ("ySize", C.c_int32), ("yBufSize", C.c_int32), ("rowDispSize", C.c_int32), ("weights", Mat), ("avgGrad", Mat),
                ("grad", Mat), ("gradRowSum2", C.c_void_p), ("weightsRowSum2", C.c_void_p), ("rowScale", C.c_void_p), ("rowDisp", C.c_void_p),
                ("sumWeight", C.c_void_p), ("sparsity", C.c_void_p), ("fast", Mat), ("fastType", C.c_int32), ("matrixScale", C.c_void_p),
                ("convertMult", C.c_void_p)]


@pytest.fixture(scope="module")
def L():
    from tscale2_amd import lib
    lib.load()
    return lib


@pytest.fixture(scope="module")
def orc():
    o = Oracle()
    o.lib.orc_apply_delta.restype = C.c_double
    return o


def mat(t):
    return Mat(t.data_ptr(), t.stride(0) * t.element_size(), t.shape[1], t.shape[0])


def packed_delta(orc, r, ys, xs):
    data = (r.standard_normal((ys, xs)) * np.exp(r.standard_normal((ys, 1)) * 1.5)).astype(np.float32)
    data[2] = 0
    q = np.zeros((ys, xs), np.int8); ts = np.zeros((xs // 128, ys), np.float32)
    orc.lib.orc_compress_delta(_ptr(data), _ptr(q), _ptr(ts), ys, xs)
    return q, ts


class DevMatrix:
    def __init__(self, w0, row_disp_size, fast_type, sparsity, with_grad):
        ys, xs = w0.shape
        ybuf = (ys + 127) // 128 * 128
        dev = "cuda"
        self.t = {"weights": torch.from_numpy(w0.copy()).cuda(), "avgGrad": torch.zeros((ys, xs), device=dev),
                  "grad": torch.zeros((ys, xs), device=dev) if with_grad else None, "gradRowSum2": torch.zeros(ys, device=dev),
                  "weightsRowSum2": torch.zeros(ys, device=dev), "rowScale": torch.zeros(ys, device=dev), "rowDisp": torch.zeros(row_disp_size, device=dev),
                  "sumWeight": torch.zeros(1, device=dev), "sparsity": torch.full((1,), sparsity, device=dev),
                  "fast": torch.full((ybuf, xs), 55, dtype=torch.int8 if fast_type == 0 else torch.uint8, device=dev),
                  "matrixScale": torch.zeros(1, device=dev), "convertMult": torch.zeros(1, device=dev)}
        t = self.t
        self.c = OptMatrix(xs, ys, ybuf, row_disp_size, mat(t["weights"]), mat(t["avgGrad"]), mat(t["grad"]) if with_grad else Mat(None, 0, 0, 0),
                           t["gradRowSum2"].data_ptr(), t["weightsRowSum2"].data_ptr(), t["rowScale"].data_ptr(), t["rowDisp"].data_ptr(),
                           t["sumWeight"].data_ptr(), t["sparsity"].data_ptr(), mat(t["fast"]), fast_type, t["matrixScale"].data_ptr(),
                           t["convertMult"].data_ptr())


def check_fast(orc, dm, w_host, fast_type, ys):
    """fast weights and matrix scale = the per-matrix quantiser of the reference applied to the updated fp32 weights"""
    xs = w_host.shape[1]
    if fast_type == 0:
        want = np.zeros((ys, xs), np.int8)
        sko = orc.lib.orc_quantize_matrix_i8(_ptr(w_host), _ptr(want), ys, xs)
    else:
        want = np.zeros((ys, xs), np.uint8)
        sko = None
    got = dm.t["fast"].cpu().numpy()
    assert (got[ys:] == 0).all()                                              # the padding rows of the fast matrix are cleared
    dev_sko = float(dm.t["matrixScale"].item())
    true_sko = float(np.sqrt((w_host.astype(np.float64) ** 2).mean()))
    assert abs(dev_sko - true_sko) <= 2e-6 * true_sko
    if fast_type == 0:
        assert abs(dev_sko - sko) <= 2e-6 * sko
        dd = np.abs(got[:ys].astype(np.int32) - want)
        assert dd.max() <= 1 and (dd != 0).mean() < 2e-3                      # the same bytes but for values within an ulp of a tie
    else:
        tab = orc.e4m3_table(hw=True)
        mult = np.float32(1) / (np.float32(dev_sko) * np.float32(1 / 32))
        wq = np.zeros((ys, xs), np.float32)
        orc.lib.orc_round_e4m3_rne(_ptr(wq), _ptr(np.ascontiguousarray(w_host * mult)), C.c_long(ys * xs))
        bad = tab[got[:ys]] != wq
        assert bad.mean() < 2e-3


@pytest.mark.parametrize("ys,xs,row_disp,fast_type", [(300, 512, 300, 0), (256, 2048, 4, 1), (70, 128, 70, 1), (384, 3072, 384, 0)])
def test_apply_one_packed_delta(L, orc, ys, xs, row_disp, fast_type):
    print("case optimiser apply", ys, xs, row_disp, fast_type, flush=True)
    r = np.random.default_rng(50 + ys)
    w0 = (r.standard_normal((ys, xs)) * 0.05).astype(np.float32)
    st = Step(0.01, 0.1, 0.9, 0.3, 0.7, 0.95)
    params = torch.tensor([st.dispDecay, st.beta1, st.weight0, st.weight1, st.l2Reg, st.rate], device="cuda")  # TAddGradientKernelParams order
    dm = DevMatrix(w0, row_disp, fast_type, 0.5, with_grad=False)
    w = w0.copy(); ag = np.zeros_like(w); rd = np.zeros(row_disp, np.float32); sw = np.zeros(1, np.float32)
    for it in range(3):                                                        # three steps: the moving statistics carry over
        q, ts = packed_delta(orc, r, ys, xs)
        qd = torch.from_numpy(q).cuda(); tsd = torch.from_numpy(ts).cuda()
        mq, mt = mat(qd), mat(tsd)
        rc = L.load().dll.ts2_opt_add_delta(C.byref(dm.c), C.byref(mq), C.byref(mt), 2, C.c_void_p(params.data_ptr()), L.load().stream())
        assert rc == 0
        torch.cuda.synchronize()
        dense = np.zeros((ys, xs), np.float32)
        orc.lib.orc_unpack_delta(_ptr(q), _ptr(ts), _ptr(dense), ys, xs, 0)
        rs = np.zeros(ys, np.float32)
        s2 = orc.lib.orc_apply_delta(_ptr(w), _ptr(ag), _ptr(dense), ys, xs, row_disp, _ptr(rd), _ptr(sw), C.c_float(0.5), C.byref(st), _ptr(rs))
        np.testing.assert_allclose(dm.t["rowScale"].cpu().numpy(), rs, rtol=1e-5)
        np.testing.assert_allclose(dm.t["rowDisp"].cpu().numpy(), rd, rtol=1e-5)
        np.testing.assert_allclose(dm.t["sumWeight"].cpu().numpy(), sw, rtol=1e-6)
        np.testing.assert_allclose(dm.t["avgGrad"].cpu().numpy(), ag, rtol=1e-5, atol=1e-6 * np.abs(ag).max())
        np.testing.assert_allclose(dm.t["weights"].cpu().numpy(), w, rtol=1e-5, atol=1e-6 * np.abs(w).max())
        np.testing.assert_allclose(dm.t["weightsRowSum2"].cpu().numpy().sum(dtype=np.float64), s2, rtol=1e-5)
        check_fast(orc, dm, dm.t["weights"].cpu().numpy(), fast_type, ys)


def test_accumulate_then_apply_equals_the_sum_applied_at_once(L, orc):
    """two packed deltas added into the fp32 gradient (UnpackDeltaKernel<0>, <1>), the second call also applying: the same as the
    oracle's step on the sum; every kernel of the sequence also checked on its own"""
    print("case optimiser accumulate", flush=True)
    ys, xs = 200, 1024
    r = np.random.default_rng(61)
    w0 = (r.standard_normal((ys, xs)) * 0.05).astype(np.float32)
    st = Step(0.02, 0.0, 0.8, 1.0, 0.5, 0.9)
    params = torch.tensor([st.dispDecay, st.beta1, st.weight0, st.weight1, st.l2Reg, st.rate], device="cuda")
    dm = DevMatrix(w0, ys, 0, 1.0, with_grad=True)
    dll = L.load().dll
    stream = L.load().stream()
    dense = np.zeros((ys, xs), np.float32)
    for it, mode in enumerate((0, 1 | 2)):                                     # store; then add + apply
        q, ts = packed_delta(orc, r, ys, xs)
        qd = torch.from_numpy(q).cuda(); tsd = torch.from_numpy(ts).cuda()
        mq, mt = mat(qd), mat(tsd)
        assert dll.ts2_opt_add_delta(C.byref(dm.c), C.byref(mq), C.byref(mt), mode, C.c_void_p(params.data_ptr()), stream) == 0
        orc.lib.orc_unpack_delta(_ptr(q), _ptr(ts), _ptr(dense), ys, xs, it)
    torch.cuda.synchronize()
    # one product and one add per element (fused into one rounding on the device)
    np.testing.assert_allclose(dm.t["grad"].cpu().numpy(), dense, rtol=0, atol=2e-7 * np.abs(dense).max())
    np.testing.assert_allclose(dm.t["gradRowSum2"].cpu().numpy(), (dense.astype(np.float64) ** 2).sum(1), rtol=2e-6)
    w = w0.copy(); ag = np.zeros_like(w); rd = np.zeros(ys, np.float32); sw = np.zeros(1, np.float32)
    orc.lib.orc_apply_delta(_ptr(w), _ptr(ag), _ptr(dense), ys, xs, ys, _ptr(rd), _ptr(sw), C.c_float(1.0), C.byref(st), None)
    np.testing.assert_allclose(dm.t["weights"].cpu().numpy(), w, rtol=1e-5, atol=1e-6 * np.abs(w).max())
    np.testing.assert_allclose(dm.t["avgGrad"].cpu().numpy(), ag, rtol=1e-5, atol=1e-6 * np.abs(ag).max())
    check_fast(orc, dm, dm.t["weights"].cpu().numpy(), 0, ys)
    # ts2_opt_convert alone (the conversion after master weights are loaded)
    dm.t["weights"].copy_(torch.from_numpy(w0))
    assert dll.ts2_opt_convert(C.byref(dm.c), stream) == 0
    torch.cuda.synchronize()
    check_fast(orc, dm, w0, 0, ys)
    # a zero matrix converts to zero bytes and scale 0
    dm.t["weights"].zero_()
    assert dll.ts2_opt_convert(C.byref(dm.c), stream) == 0
    torch.cuda.synchronize()
    assert (dm.t["fast"].cpu().numpy() == 0).all() and float(dm.t["matrixScale"].item()) == 0.0
