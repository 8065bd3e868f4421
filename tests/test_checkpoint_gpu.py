"""A checkpoint written by the reference's own classes carried into the device model and through a step (the reason the checkpoint format is
on the path: src/gpt/train/main_gpt.cpp:528-535 loads TModelParams and hands every matrix to the compute context).
tests/golden/ref_golden.npz: `checkpoint.e128` = SAVELOAD bytes of a TModelParams laid out by the reference for the model string
e128h1d1ffn1w16 (tests/golden/make_golden.py); ts2_checkpoint_parse -> ts2_model_set_master for every matrix -> one step."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")
from model_harness import E4M3, I8, NO_SCALE, Harness, QMatrix, rel_err, scale_fit  # noqa: E402
from test_checkpoint import Info, MatView  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = np.load(os.path.join(ROOT, "tests", "golden", "ref_golden.npz"))


@pytest.mark.parametrize("mode", [I8, E4M3])
def test_checkpoint_bytes_to_device_model_and_through_a_step(mode):
    print("case checkpoint -> device -> step", mode, flush=True)
    from tscale2_amd import lib as L
    lib = L.load()
    dll = lib.dll
    dll.ts2_checkpoint_parse.restype = C.c_void_p
    raw = GOLD["checkpoint.e128"]
    ck = dll.ts2_checkpoint_parse(raw.ctypes.data_as(C.c_void_p), C.c_int64(raw.size))
    assert ck
    ck = C.c_void_p(ck)
    try:
        info = Info()
        assert dll.ts2_checkpoint_get_info(ck, C.byref(info)) == 0
        assert (info.dim, info.headCount, info.ffnTiles, info.moeExpertCount) == (128, 1, 1, 0)
        vocab = int(info.outputTokenCount)
        # the schedule and the attention types as the checkpoint holds them = what the library derives from the depth
        lt, la, ls, aw = [], [], [], []
        for d in range(info.layerCount):
            t, sl, aid, mc = C.c_int32(), C.c_float(), C.c_int32(), C.c_int32()
            assert dll.ts2_checkpoint_layer(ck, d, C.byref(t), C.byref(sl), C.byref(aid), C.byref(mc)) == 0
            lt.append(t.value); la.append(aid.value); ls.append(sl.value)
        for a in range(info.attTypeCount):
            w, ty = C.c_int32(), C.c_int32()
            assert dll.ts2_checkpoint_att_type(ck, a, C.byref(w), C.byref(ty)) == 0
            aw.append(w.value)
        slt, sla, sls, saw = L.model_schedule(info.depth, 0, aw[-1])
        assert lt == list(slt) and la == list(sla) and ls == list(sls) and aw == list(saw)

        def weights(layer, mid):
            v = MatView()
            assert dll.ts2_checkpoint_matrix(ck, layer, mid, C.byref(v)) == 0
            return np.ctypeslib.as_array(v.weights, (v.ySize, v.xSize)).copy(), v.rowDispSize, v.sparsity
        bias = np.ctypeslib.as_array(info.bias, (info.biasCount,)).copy()
        # the same model for the CPU side: a harness whose matrices are the checkpoint's
        h = Harness(mode, dim=info.dim, heads=info.headCount, ffn_tiles=info.ffnTiles, depth=info.depth, vocab=vocab, frag_count=4, frag_len=64,
                    wide_window=aw[-1], seed=31)
        assert list(h.lt) == lt and list(h.la) == la
        ck_mats = []
        for d in range(h.depth):
            for i in range(len(h.layers[d])):
                w, rds, sp = weights(d, i)
                assert w.shape == h.layers[d][i].w.shape
                h.layers[d][i] = QMatrix(h.orc, w, mode, i in NO_SCALE[int(h.lt[d])])
                ck_mats.append((d, i, h.layers[d][i], rds, sp))
        w, rds, sp = weights(-1, 0)
        h.embed = QMatrix(h.orc, w, mode, False); ck_mats.append((L.LAYER_EMBED, 0, h.embed, rds, sp))
        w, rds, sp = weights(-1, 1)
        h.final = QMatrix(h.orc, w, mode, False); ck_mats.append((L.LAYER_FINAL, 0, h.final, rds, sp))
        h.bias = bias
    finally:
        dll.ts2_checkpoint_free(ck)
    bdt = np.int8 if mode == I8 else np.uint8
    # ---- device model A: every parsed matrix through ts2_model_set_master (fp32 master -> fast weights on the device)
    m = h.device_model()
    try:
        fast = []
        for d, i, q, rds, sp in ck_mats:
            m.set_master(d, i, q.w, rds, sp)
            assert np.array_equal(m.get_master(d, i, *q.w.shape), q.w)                      # the checkpoint's floats, in place
            f, scale = m.get_matrix(d, i, *q.fast.shape, bdt)
            assert abs(scale - q.scale) <= 3e-6 * q.scale                                   # the per-matrix quantiser of quant.h:42-62
            assert (f != q.fast).mean() < 2e-3                                              # (values within an ulp of a rounding tie)
            fast.append((f, scale))
        m.backprop()
        torch.cuda.synchronize()
        loss_a = m.loss_sum()
        got = [m.get_delta(d, i, *q.fast.shape) for d, i, q, _, _ in ck_mats] + [m.array("stateGrad").float().cpu().numpy()]
    finally:
        m.close()
    # ---- device model B: a fresh model that is handed the same fast weights: the step must be the same bit for bit
    m2 = h.device_model()
    try:
        for (d, i, q, _, _), (f, scale) in zip(ck_mats, fast):
            m2.set_matrix(d, i, f, scale)
        m2.backprop()
        torch.cuda.synchronize()
        assert abs(m2.loss_sum() - loss_a) <= 2e-6 * abs(loss_a)                            # (summed with fp32 atomics)
        want = [m2.get_delta(d, i, *q.fast.shape) for d, i, q, _, _ in ck_mats] + [m2.array("stateGrad").float().cpu().numpy()]
    finally:
        m2.close()
    for (d, i, _, _, _), g, w in zip(ck_mats + [("stateGrad", 0, None, 0, 0)], got, want):
        if d == L.LAYER_EMBED:   # the embedding delta is summed with fp32 atomics: equal up to the order of the additions
            np.testing.assert_allclose(g, w, rtol=0, atol=1e-6 * np.abs(w).max())
        else:
            assert np.array_equal(g, w), (d, i)
    # ---- and against the CPU oracle's step on the harness' dequantised copies of the same weights (8-bit storage noise: statistical)
    h.oracle_step()
    n_t = (h.target >= 0).sum()
    print("loss", loss_a / n_t, h.ref_loss, flush=True)
    assert abs(loss_a / n_t - h.ref_loss) <= 5e-3 * abs(h.ref_loss)
    k = 0
    for d in range(h.depth):
        for i in range(len(h.layers[d])):
            fit, corr = scale_fit(got[k], h.ref_delta[d][i])
            rms, _ = rel_err(got[k], h.ref_delta[d][i])
            print(f"layer {d} matrix {i}: rms {rms:.3f} fit {fit:.4f} corr {corr:.4f}", flush=True)
            assert abs(fit - 1) <= 2e-2 and corr >= 0.98, (d, i, fit, corr)
            k += 1
