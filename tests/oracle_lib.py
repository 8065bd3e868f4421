"""ctypes bindings of the CPU oracle (oracle/liboracle.so) and, where it was built, of the reference's own CPU sources
(oracle/_ref/libts2ref.so).  Test infrastructure: only tests, the smoke check and the benchmark's cpu_baseline leg use it."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "liboracle.so")
REF_SO = os.path.join(ORACLE_DIR, "_ref", "libts2ref.so")

F32 = np.float32
fp = C.POINTER(C.c_float)
ip = C.POINTER(C.c_int)


def _ptr(a, t=None):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be contiguous"
    return a.ctypes.data_as(C.c_void_p)


def load_oracle():
    if not os.path.exists(ORACLE_SO):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "liboracle.so"])
    lib = C.CDLL(ORACLE_SO)
    lib.orc_e4m3_to_float.restype = C.c_float
    lib.orc_e4m3_to_float.argtypes = [C.c_int]
    lib.orc_cvt_i8.restype = C.c_int8
    lib.orc_cvt_i8.argtypes = [C.c_float]
    lib.orc_cvt_e4m3.restype = C.c_uint8
    lib.orc_cvt_e4m3.argtypes = [C.c_float]
    lib.orc_cvt_e4m3_rne.restype = C.c_uint8
    lib.orc_cvt_e4m3_rne.argtypes = [C.c_float]
    lib.orc_quantize_matrix_i8.restype = C.c_float
    lib.orc_quantize_matrix_e4m3.restype = C.c_float
    lib.orc_grad_mult.restype = C.c_float
    lib.orc_grad_mult.argtypes = [C.c_float]
    lib.orc_bf16_round.restype = C.c_float
    lib.orc_bf16_round.argtypes = [C.c_float]
    lib.orc_model_step.restype = C.c_double
    return lib


def load_ref():
    """The reference's own CPU code; None where it has not been built (it needs the reference tree at build time)."""
    if not os.path.exists(REF_SO):
        return None
    lib = C.CDLL(REF_SO)
    lib.ref_e4m3_to_float.restype = C.c_float
    lib.ref_e4m3_to_float.argtypes = [C.c_int]
    return lib


class OrcDims(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("dim", "qDim", "ttDim", "headCount", "ffnDim", "expertDim", "expertCount", "moeSelected")]


class OrcLayer(C.Structure):
    _fields_ = [("type", C.c_int), ("alibiSlope", C.c_float), ("attTypeId", C.c_int), ("w", C.c_void_p * 5), ("delta", C.c_void_p * 5)]


class OrcCommon(C.Structure):
    _fields_ = [("attTypeCount", C.c_int), ("spanPtr", C.c_void_p * 4), ("spans", C.c_void_p * 4), ("revPtr", C.c_void_p * 4),
                ("revSpans", C.c_void_p * 4), ("ropeBuf", C.c_void_p)]


class Oracle:
    """numpy-level API over liboracle.so (or over libts2ref.so for the functions both export, with use_ref=True)."""

    def __init__(self, use_ref=False):
        self.use_ref = use_ref
        self.lib = load_ref() if use_ref else load_oracle()
        if self.lib is None:
            raise FileNotFoundError(REF_SO)
        self.p = "ref_" if use_ref else "orc_"

    def _f(self, name):
        return getattr(self.lib, self.p + name)

    # ---- linalg
    def mul_forward(self, vec, kqv):
        vec = np.ascontiguousarray(vec, F32); kqv = np.ascontiguousarray(kqv, F32)
        len_, dim = vec.shape; rdim = kqv.shape[0]
        res = np.empty((len_, rdim), F32)
        self._f("mul_forward")(_ptr(vec), _ptr(kqv), _ptr(res), len_, dim, rdim)
        return res

    def mul_backward_accum(self, vec_grad, kqv, res_grad):
        g = np.array(vec_grad, F32, order="C"); kqv = np.ascontiguousarray(kqv, F32); r = np.ascontiguousarray(res_grad, F32)
        len_, dim = g.shape; rdim = kqv.shape[0]
        self._f("mul_backward_accum")(_ptr(g), _ptr(kqv), _ptr(r), len_, dim, rdim)
        return g

    def sum_rank_one(self, vec, res_grad):
        vec = np.ascontiguousarray(vec, F32); r = np.ascontiguousarray(res_grad, F32)
        len_, dim = vec.shape; rdim = r.shape[1]
        d = np.empty((rdim, dim), F32)
        self._f("sum_rank_one")(_ptr(vec), _ptr(d), _ptr(r), len_, dim, rdim)
        return d

    # ---- norm / lolu
    def normalize_state(self, state, head_count):
        s = np.ascontiguousarray(state, F32); res = np.empty_like(s)
        self._f("normalize_state")(_ptr(s), _ptr(res), s.shape[0], s.shape[1], head_count)
        return res

    def normalize_state_backward(self, state, dnorm, head_count):
        s = np.ascontiguousarray(state, F32); d = np.ascontiguousarray(dnorm, F32); g = np.empty_like(s)
        self._f("normalize_state_backward")(_ptr(s), _ptr(d), _ptr(g), s.shape[0], s.shape[1], head_count)
        return g

    def lolu(self, gate, vals):
        g = np.ascontiguousarray(gate, F32); v = np.ascontiguousarray(vals, F32); r = np.empty_like(g)
        self._f("lolu")(_ptr(g), _ptr(v), _ptr(r), g.shape[0], g.shape[1])
        return r

    def backprop_lolu(self, gate, vals, grad):
        g = np.ascontiguousarray(gate, F32); v = np.ascontiguousarray(vals, F32); d = np.ascontiguousarray(grad, F32)
        gg = np.empty_like(g); gv = np.empty_like(g)
        self._f("backprop_lolu")(_ptr(g), _ptr(v), _ptr(d), _ptr(gg), _ptr(gv), g.shape[0], g.shape[1])
        return gg, gv

    # ---- rope / attention
    def fill_rope_buf(self, width, rope_len):
        buf = np.empty((rope_len, width), F32)
        self._f("fill_rope_buf")(_ptr(buf), width, rope_len)
        return buf

    def apply_rope(self, rope_buf, direction, p):
        r = np.ascontiguousarray(rope_buf, F32); v = np.array(p, F32, order="C")
        if self.use_ref:
            self.lib.ref_apply_rope(_ptr(r), r.shape[1], r.shape[0], C.c_float(direction), _ptr(v), v.shape[0], v.shape[1])
        else:
            self.lib.orc_apply_rope(_ptr(r), r.shape[1], C.c_float(direction), _ptr(v), v.shape[0], v.shape[1])
        return v

    def transpose_attention(self, span_ptr, spans):
        span_ptr = np.ascontiguousarray(span_ptr, np.int32); spans = np.ascontiguousarray(spans, np.int32).reshape(-1, 2)
        n = len(span_ptr) - 1
        edges = int((spans[:, 1] - spans[:, 0] + 1).sum()) if len(spans) else 0
        rp = np.zeros(n + 1, np.int32); rs = np.zeros((max(edges, 1), 2), np.int32)
        cnt = self._f("transpose_attention")(n, _ptr(span_ptr), _ptr(spans), _ptr(rp), _ptr(rs), max(edges, 1))
        assert cnt >= 0
        return rp, rs[:cnt].copy()

    def attention(self, heads, qdim, ttdim, slope, span_ptr, spans, q, k, v, dval=None, att_scale_mult=1.0):
        """Forward (+ backward when dval is given).  Returns dict of arrays."""
        span_ptr = np.ascontiguousarray(span_ptr, np.int32); spans = np.ascontiguousarray(spans, np.int32).reshape(-1, 2)
        q = np.ascontiguousarray(q, F32); k = np.ascontiguousarray(k, F32); v = np.ascontiguousarray(v, F32)
        n = q.shape[0]
        val = np.zeros((n, heads * ttdim), F32); sw = np.zeros((heads, n), F32); mx = np.zeros((heads, n), F32)
        out = {"val": val, "sum_weight": sw, "max_dp": mx}
        if dval is not None:
            dval = np.ascontiguousarray(dval, F32)
            ds = np.zeros((heads, n), F32); dq = np.zeros_like(q); dk = np.zeros_like(k); dv = np.zeros_like(v)
            out.update(dscale=ds, dq=dq, dk=dk, dv=dv)
        if self.use_ref:
            self.lib.ref_attention(n, heads, qdim, ttdim, C.c_float(slope), C.c_float(att_scale_mult), _ptr(span_ptr), _ptr(spans),
                                   _ptr(q), _ptr(k), _ptr(v), _ptr(dval), _ptr(val), _ptr(sw), _ptr(mx),
                                   _ptr(out.get("dscale")), _ptr(out.get("dq")), _ptr(out.get("dk")), _ptr(out.get("dv")))
            return out
        L = self.lib
        sl, am = C.c_float(slope), C.c_float(att_scale_mult)
        L.orc_attention_forward(n, heads, qdim, ttdim, sl, am, _ptr(span_ptr), _ptr(spans), _ptr(q), _ptr(k), _ptr(v), _ptr(val), _ptr(sw), _ptr(mx))
        if dval is not None:
            rp, rs = self.transpose_attention(span_ptr, spans)
            rs = np.ascontiguousarray(rs) if len(rs) else np.zeros((1, 2), np.int32)
            L.orc_compute_dscale(n, heads, ttdim, _ptr(val), _ptr(dval), _ptr(ds))
            L.orc_attention_grad_q(n, heads, qdim, ttdim, sl, am, _ptr(span_ptr), _ptr(spans), _ptr(q), _ptr(k), _ptr(v), _ptr(dval),
                                   _ptr(ds), _ptr(sw), _ptr(mx), _ptr(dq))
            L.orc_attention_grad_k(n, heads, qdim, ttdim, sl, am, _ptr(rp), _ptr(rs), _ptr(q), _ptr(k), _ptr(v), _ptr(dval),
                                   _ptr(ds), _ptr(sw), _ptr(mx), _ptr(dk), _ptr(dv))
        return out

    def make_causal_spans(self, frag_count, frag_len, window):
        n = frag_count * frag_len
        sp = np.zeros(n + 1, np.int32); spans = np.zeros((n, 2), np.int32); cnt = C.c_int(0)
        self.lib.orc_make_causal_spans(frag_count, frag_len, window, _ptr(sp), _ptr(spans), C.byref(cnt))
        return sp, spans[:cnt.value].copy()

    # ---- model schedule / batch nodes
    def model_schedule(self, descr, depth, experts, wide_window):
        """layer schedule {type, attention type id, slope} and attention widths.  Reference side: parsed from the model string by
        InitModelDescrImpl; oracle side: orc_model_schedule from the numbers the string stands for (the caller supplies both)."""
        lt = np.zeros(256, np.int32); la = np.zeros(256, np.int32); ls = np.zeros(256, F32); aw = np.zeros(8, np.int32); ac = C.c_int(0)
        out = {}
        if self.use_ref:
            dims = np.zeros(10, np.int32)
            n = self.lib.ref_model_descr(descr.encode(), _ptr(dims), _ptr(lt), _ptr(la), _ptr(ls), 256, _ptr(aw), C.byref(ac))
            out["dims"] = dims
        else:
            n = self.lib.orc_model_schedule(depth, experts, wide_window, _ptr(lt), _ptr(la), _ptr(ls), 256, _ptr(aw), C.byref(ac))
        assert n > 0
        out.update(layer_type=lt[:n].copy(), layer_att_id=la[:n].copy(), layer_slope=ls[:n].copy(), att_width=aw[:ac.value].copy())
        return out

    def ref_label_data(self, descr, vocab, tokens, targets, att_type):
        """InitLabelData of the reference build (noise labels disabled) for equal-length fragments: tokens/targets [frag][len]"""
        assert self.use_ref
        tokens = np.ascontiguousarray(tokens, np.int32); targets = np.ascontiguousarray(targets, np.int32)
        fc, fl = tokens.shape
        n = fc * fl
        lc = C.c_int(0); tc = C.c_int(0)
        lp = np.zeros(n + 1, np.int32); lb = np.zeros(4 * n, np.uint32); tp = np.zeros((n, 2), np.int32)
        sp = np.zeros(n + 1, np.int32); ss = np.zeros((4 * n, 2), np.int32)
        got = self.lib.ref_init_label_data(descr.encode(), vocab, fc, fl, _ptr(tokens), _ptr(targets), C.byref(lc), _ptr(lp), _ptr(lb), C.byref(tc),
                                           _ptr(tp), att_type, _ptr(sp), _ptr(ss))
        assert got == n
        return {"label_count": np.array([lc.value], np.int32), "label_ptr": lp, "labels": lb[:lp[n]].copy(), "target_pairs": tp[:tc.value].copy(),
                "span_ptr": sp, "spans": ss[:sp[n]].copy()}

    # ---- converters
    def convert_i8(self, src, mult):
        s = np.ascontiguousarray(src, F32).ravel(); d = np.empty(s.size, np.int8)
        self._f("convert_i8")(_ptr(d), _ptr(s), s.size, C.c_float(mult))
        return d.reshape(np.shape(src))

    def convert_e4m3(self, src, mult):
        s = np.ascontiguousarray(src, F32).ravel(); d = np.empty(s.size, np.uint8)
        self._f("convert_e4m3")(_ptr(d), _ptr(s), s.size, C.c_float(mult))
        return d.reshape(np.shape(src))

    def e4m3_table(self, hw=False):
        """code -> value.  hw=True gives the hardware (OCP) reading of code 0x80 as -0; the reference's slow decoder
        (src/util/fp8.h:4-21) only special-cases code 0 and reads 0x80 as -2^-7, a code its own encoder never emits."""
        tab = np.array([self._f("e4m3_to_float")(c) for c in range(256)], F32)
        if hw:
            tab[0x80] = -0.0
        return tab
