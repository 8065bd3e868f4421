"""Checkpoint and weight-exchange formats (host code of the library, no GPU) against bytes the reference's own classes wrote:
tests/golden/ref_golden.npz holds two TModelParams serialised by its SAVELOAD / bin_saver (laid out for a dense and a MoE model string by
its own InitModelDescr / EnumLayerMatrices; src/gpt/model_params/model_params.h:7-18) and a matrix in its fp16-row wire format together
with the result of its AddPackedMatrix (model_matrix.cpp:6-58)."""
import ctypes as C
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = np.load(os.path.join(ROOT, "tests", "golden", "ref_golden.npz"))


class Info(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("dim", "qDim", "ttDim", "expertDim", "headCount", "ffnTiles", "moeExpertCount", "moeSelected", "kvRep", "depth")] + \
               [(n, C.c_int64) for n in ("labelCount", "inputTokenCount", "outputTokenCount")] + [("attTypeCount", C.c_int32), ("layerCount", C.c_int32),
                ("flags", C.c_uint64), ("docStartToken", C.c_uint64), ("fragLen", C.c_int64), ("biasCount", C.c_int32), ("bias", C.POINTER(C.c_float))]


class MatView(C.Structure):
    _fields_ = [("xSize", C.c_int32), ("ySize", C.c_int32), ("weights", C.POINTER(C.c_float)), ("avgGrad", C.POINTER(C.c_float)), ("sumWeight", C.c_float),
                ("rowDisp", C.POINTER(C.c_float)), ("rowDispSize", C.c_int32), ("sparsity", C.c_float)]


@pytest.fixture(scope="module")
def dll():
    d = C.CDLL(os.path.join(ROOT, "tscale2_amd", "libts2amd.so"))
    d.ts2_checkpoint_parse.restype = C.c_void_p
    d.ts2_checkpoint_write.restype = C.c_int64
    d.ts2_pack_matrix_fp16.restype = C.c_int64
    return d


@pytest.mark.parametrize("name,descr", [("dense", "e16h1d3ffn1w16"), ("moe", "e32xp128moe2moes1h2d1w48")])
def test_checkpoint_parses_and_writes_back_byte_for_byte(dll, name, descr):
    from model_harness import parse_model_descr
    from oracle_lib import Oracle
    raw = GOLD["checkpoint." + name]
    ck = dll.ts2_checkpoint_parse(raw.ctypes.data_as(C.c_void_p), C.c_int64(raw.size))
    assert ck
    ck = C.c_void_p(ck)
    try:
        info = Info()
        assert dll.ts2_checkpoint_get_info(ck, C.byref(info)) == 0
        dims, wide = parse_model_descr(descr)
        got_dims = [info.dim, info.qDim, info.ttDim, info.expertDim, info.headCount, info.ffnTiles, info.moeExpertCount, info.moeSelected, info.kvRep, info.depth]
        assert got_dims == list(dims)
        vocab = 32 if name == "dense" else 20
        assert (info.labelCount, info.inputTokenCount, info.outputTokenCount) == (vocab + 1, vocab, vocab)
        assert info.biasCount == vocab
        np.testing.assert_allclose(np.ctypeslib.as_array(info.bias, (vocab,)), 0.01 * np.arange(vocab), rtol=1e-6)
        # layer schedule and attention types = what the model string stands for (pinned against the reference's parser elsewhere)
        sched = Oracle().model_schedule(descr, int(dims[9]), int(dims[6]), wide)
        assert info.layerCount == len(sched["layer_type"]) and info.attTypeCount == len(sched["att_width"])
        for a in range(info.attTypeCount):
            w, t = C.c_int32(), C.c_int32()
            assert dll.ts2_checkpoint_att_type(ck, a, C.byref(w), C.byref(t)) == 0
            assert (w.value, t.value) == (int(sched["att_width"][a]), 0)
        # every matrix: shapes of EnumLayerMatrices, the seeded fill in storage order, the optimiser state that was set
        state = 7
        q, tt, dim, ffn, xp, experts = 128 * dims[4], 128 * dims[4], dims[0], 128 * dims[5], dims[3], dims[6]
        shapes = {0: [(dim, q)] * 4 + [(tt, dim)], 2: [(dim, ffn), (dim, ffn), (ffn, dim)],
                  3: [(dim, xp * experts), (dim, xp * experts), (xp, dim * experts), (dim, experts)]}  # (xSize, ySize)

        def check_matrix(layer, mid, xs, ys):
            nonlocal state
            v = MatView()
            assert dll.ts2_checkpoint_matrix(ck, layer, mid, C.byref(v)) == 0
            assert (v.xSize, v.ySize) == (xs, ys), (layer, mid, v.xSize, v.ySize)
            w = np.ctypeslib.as_array(v.weights, (ys, xs)); g = np.ctypeslib.as_array(v.avgGrad, (ys, xs))
            want_w = np.zeros((ys, xs), np.float32); want_g = np.zeros((ys, xs), np.float32)
            for i in range(ys * xs):
                state = (state * 1664525 + 1013904223) & 0xffffffff
                want_w.flat[i] = np.float32(((state >> 8) % 2001 - 1000) * np.float32(1 / 1024))
                state = (state * 1664525 + 1013904223) & 0xffffffff
                want_g.flat[i] = np.float32(np.float32(((state >> 8) % 2001 - 1000) * np.float32(1 / 1024)) * np.float32(0.25))
            assert np.array_equal(w, want_w) and np.array_equal(g, want_g)
            return v
        v = check_matrix(-1, 0, dim, vocab + 1)
        assert v.rowDispSize == vocab + 1 and v.sparsity == 1.0                     # SetSizesPerRowDisp
        v = check_matrix(-1, 1, dim, vocab)
        assert v.rowDispSize == vocab and v.sumWeight == 2.5
        np.testing.assert_array_equal(np.ctypeslib.as_array(v.rowDisp, (vocab,)), 0.125 + np.arange(vocab, dtype=np.float32))
        for d in range(info.layerCount):
            lt, sl, aid, mc = C.c_int32(), C.c_float(), C.c_int32(), C.c_int32()
            assert dll.ts2_checkpoint_layer(ck, d, C.byref(lt), C.byref(sl), C.byref(aid), C.byref(mc)) == 0
            assert (lt.value, aid.value) == (int(sched["layer_type"][d]), int(sched["layer_att_id"][d])) and sl.value == float(sched["layer_slope"][d])
            assert mc.value == len(shapes[lt.value])
            for i, (xs, ys) in enumerate(shapes[lt.value]):
                v = check_matrix(d, i, xs, ys)
                assert v.rowDispSize == 1                                               # SetSizesPerMatrixDisp
                if d == 0 and i == 0:
                    assert v.sumWeight == 1.5 and v.rowDisp[0] == 0.75
        # written back: the same bytes; a short buffer is not overrun and the size needed is reported
        n = dll.ts2_checkpoint_write(ck, None, C.c_int64(0))
        assert n == raw.size
        out = np.full(raw.size + 16, 0xAB, np.uint8)
        assert dll.ts2_checkpoint_write(ck, out.ctypes.data_as(C.c_void_p), C.c_int64(raw.size)) == raw.size
        assert np.array_equal(out[:raw.size], raw) and (out[raw.size:] == 0xAB).all()
        short = np.full(100, 0xAB, np.uint8)
        assert dll.ts2_checkpoint_write(ck, short.ctypes.data_as(C.c_void_p), C.c_int64(50)) == raw.size and (short[50:] == 0xAB).all()
    finally:
        dll.ts2_checkpoint_free(ck)
    # truncated or padded bytes are refused
    assert not dll.ts2_checkpoint_parse(raw.ctypes.data_as(C.c_void_p), C.c_int64(raw.size - 1))
    padded = np.concatenate([raw, np.zeros(4, np.uint8)])
    assert not dll.ts2_checkpoint_parse(padded.ctypes.data_as(C.c_void_p), C.c_int64(padded.size))


def test_fp16_row_wire_format_matches_the_reference_bytes(dll):
    m = np.ascontiguousarray(GOLD["wire.matrix"]); packed = GOLD["wire.packed"]
    ys, xs = m.shape
    n = dll.ts2_pack_matrix_fp16(m.ctypes.data_as(C.c_void_p), xs, ys, None, C.c_int64(0))
    assert n == packed.size == 4 * ys + 2 * xs * (ys - 1)                            # the zero row carries its rms only
    out = np.zeros(n, np.uint8)
    assert dll.ts2_pack_matrix_fp16(m.ctypes.data_as(C.c_void_p), xs, ys, out.ctypes.data_as(C.c_void_p), C.c_int64(n)) == n
    assert np.array_equal(out, packed)
    acc = np.ascontiguousarray(GOLD["wire.base"]).copy()
    assert dll.ts2_add_packed_matrix_fp16(acc.ctypes.data_as(C.c_void_p), xs, ys, packed.ctypes.data_as(C.c_void_p), C.c_int64(packed.size), C.c_float(0.75)) == 0
    assert np.array_equal(acc.view(np.uint32), GOLD["wire.added"].view(np.uint32))
    # round trip: within half an ulp of a half relative to the row's rms (values inside the half range)
    back = np.zeros_like(m)
    dll.ts2_add_packed_matrix_fp16(back.ctypes.data_as(C.c_void_p), xs, ys, packed.ctypes.data_as(C.c_void_p), C.c_int64(packed.size), C.c_float(1.0))
    rms = np.sqrt((m.astype(np.float64) ** 2).mean(1))
    rows = [y for y in range(ys) if y != 5]
    assert (np.abs(back[rows] - m[rows]) <= 2.0 ** -11 * np.abs(m[rows]) + 2.0 ** -25 * rms[rows, None]).all()
    assert dll.ts2_add_packed_matrix_fp16(acc.ctypes.data_as(C.c_void_p), xs, ys, packed.ctypes.data_as(C.c_void_p), C.c_int64(packed.size - 2), C.c_float(1.0)) == -1
