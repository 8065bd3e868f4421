"""Harness shared by the model-level tests and the benchmark: builds a model the way the reference's own harness does
(model string -> layer schedule, src/gpt/model_params/model_dim.cpp:82-158; nodes of a batch, src/gpt/att/sliding_window.cpp:269-306
with noise labels disabled; per-matrix quantisation, src/gpt/matrix/quant.h:42-62) and feeds identical quantised weights and batches
to the CPU oracle and to the GPU step driver."""
import ctypes as C

import numpy as np

from oracle_lib import Oracle, OrcCommon, OrcDims, OrcLayer, _ptr

LT_ATT, LT_FFN, LT_MOE = 0, 2, 3
I8, E4M3 = 0, 1


def schedule(orc, depth, experts, wide_window):
    r = orc.model_schedule(None, depth, experts, wide_window)
    return r["layer_type"], r["layer_att_id"], r["layer_slope"], r["att_width"]


def parse_model_descr(descr):
    """The numbers a reference model string stands for (TModelDescrString, src/gpt/model_params/model_dim.cpp:17-58), in the order
    {Dim, QDim, TTDim, ExpertDim, HeadCount, FfnTiles, MoeExpertCount, MoeSelected, KVrep, Depth} + the wide attention window.
    Fields that a string does not name keep the reference's defaults."""
    import re
    f = {k: float(v) for k, v in re.findall(r"([a-z]+)([0-9.]+)", descr)}
    dims = [int(f.get("e", 256)), 128, 128, int(f.get("xp", 128)), int(f.get("h", 1)), int(f.get("ffn", 1)), int(f.get("moe", 0)),
            int(f.get("moes", 2)), int(f.get("rep", 16)), int(f.get("d", 60))]
    return np.array(dims, np.int32), int(f.get("w", 64))


def make_batch(orc, vocab, tokens, att_widths):
    """Nodes of a batch of equal-length fragments as InitLabelData builds them with noise labels disabled
    (src/gpt/att/sliding_window.cpp:269-306): one label 1 + token per node, target = next token of the fragment (none for the last),
    one causal span [max(fragment start, t - width), t - 1] per node and attention type."""
    tokens = np.asarray(tokens)
    frag_count, frag_len = tokens.shape
    n = frag_count * frag_len
    label_ptr = np.arange(n + 1, dtype=np.int32)
    labels = (1 + tokens).astype(np.uint32).ravel()
    tg = np.full((frag_count, frag_len), -1, np.int32)
    tg[:, :-1] = tokens[:, 1:]
    spans = [orc.make_causal_spans(frag_count, frag_len, int(w)) for w in att_widths]
    return {"label_count": vocab + 1, "label_ptr": label_ptr, "labels": labels, "target": tg.ravel(), "spans": spans}


def layer_shapes(ltype, dim, heads, ffn, xp, experts):
    """[out][in] shapes of a layer's matrices (EnumLayerMatrices, src/gpt/model_params/model_dim.h:225-262)"""
    q = heads * 128
    if ltype == LT_ATT:
        return [(q, dim), (q, dim), (q, dim), (q, dim), (dim, q)]
    if ltype == LT_FFN:
        return [(ffn, dim), (ffn, dim), (dim, ffn)]
    return [(xp * experts, dim), (xp * experts, dim), (dim * experts, xp), (experts, dim)]


NO_SCALE = {LT_ATT: {3}, LT_FFN: {1}, LT_MOE: {1, 3}}  # matrices read with GetDataNoScale (gate, select)


class QMatrix:
    """per-matrix quantised weights: fast bytes + scale, and the dequantised fp32 view the CPU path multiplies with"""

    def __init__(self, orc, w, mode, no_scale):
        rows, cols = w.shape
        w = np.ascontiguousarray(w, np.float32)
        self.w = w  # the fp32 master weights the fast bytes were derived from
        if mode == I8:
            self.fast = np.zeros((rows, cols), np.int8)
            self.scale = float(orc.lib.orc_quantize_matrix_i8(_ptr(w), _ptr(self.fast), rows, cols))
            vals = self.fast.astype(np.float32)
        else:
            self.fast = np.zeros((rows, cols), np.uint8)
            self.scale = float(orc.lib.orc_quantize_matrix_e4m3(_ptr(w), _ptr(self.fast), rows, cols))
            vals = orc.e4m3_table()[self.fast]
        s = np.float32(1 / 32) if no_scale else np.float32(1 / 32) * np.float32(self.scale)
        self.deq = np.ascontiguousarray(vals * s, np.float32)


class Harness:
    def __init__(self, mode, dim, heads, ffn_tiles, depth, vocab, frag_count, frag_len, wide_window=64, experts=0, selected=2, xp=128, seed=1,
                 std=0.02, k_std=None, bias_std=0.0, sel_std=None):
        self.orc = Oracle()
        self.mode, self.dim, self.heads, self.ffn = mode, dim, heads, ffn_tiles * 128
        self.experts, self.selected, self.xp = experts, selected, xp
        self.vocab, self.label_count = vocab, vocab + 1
        self.lt, self.la, self.ls, self.att_width = schedule(self.orc, depth, experts, wide_window)
        self.depth = len(self.lt)
        r = np.random.default_rng(seed)
        self.layers = []
        for d in range(self.depth):
            mats = []
            for i, (rows, cols) in enumerate(layer_shapes(self.lt[d], dim, heads, self.ffn, xp, experts)):
                s = std if not (k_std and self.lt[d] == LT_ATT and i == 1) else k_std
                if sel_std and self.lt[d] == LT_MOE and i == 3:
                    s = sel_std  # the select matrix: wider logit gaps, fewer tokens whose top-k choice hangs on 8-bit noise
                mats.append(QMatrix(self.orc, r.standard_normal((rows, cols)) * s, mode, i in NO_SCALE[int(self.lt[d])]))
            self.layers.append(mats)
        self.embed = QMatrix(self.orc, r.standard_normal((self.label_count, dim)) * std, mode, False)
        self.final = QMatrix(self.orc, r.standard_normal((vocab, dim)) * std, mode, False)
        # final-layer bias (log2 units); drawn from its own generator so that the other draws do not depend on it
        self.bias = (np.random.default_rng(seed + 1000).standard_normal(vocab) * bias_std).astype(np.float32)
        # batch: uniform random tokens, target = next token of the fragment, label = 1 + token (noise labels disabled)
        self.n = frag_count * frag_len
        tokens = r.integers(0, vocab, (frag_count, frag_len))
        b = make_batch(self.orc, vocab, tokens, self.att_width)
        assert b["label_count"] == self.label_count
        self.label_ptr, self.labels, self.target, self.spans = b["label_ptr"], b["labels"], b["target"], b["spans"]
        self.rev = [self.orc.transpose_attention(sp, ss) for sp, ss in self.spans]
        self.rope = self.orc.fill_rope_buf(128, self.n)

    # ---- oracle side
    def oracle_step(self, want_deltas=True):
        o = self.orc
        dims = OrcDims(self.dim, 128, 128, self.heads, self.ffn, self.xp, self.experts, self.selected)
        layers = (OrcLayer * self.depth)()
        self.ref_delta = []
        keep = []
        for d in range(self.depth):
            layers[d].type = int(self.lt[d]); layers[d].alibiSlope = float(self.ls[d]); layers[d].attTypeId = int(self.la[d])
            ds = []
            for i, m in enumerate(self.layers[d]):
                layers[d].w[i] = m.deq.ctypes.data
                dl = np.zeros_like(m.deq)
                ds.append(dl)
                layers[d].delta[i] = dl.ctypes.data if want_deltas else None
            self.ref_delta.append(ds)
        com = OrcCommon()
        com.attTypeCount = len(self.spans)
        for a, ((sp, ss), (rp, rs)) in enumerate(zip(self.spans, self.rev)):
            ss = np.ascontiguousarray(ss) if len(ss) else np.zeros((1, 2), np.int32)
            rs = np.ascontiguousarray(rs) if len(rs) else np.zeros((1, 2), np.int32)
            keep += [sp, ss, rp, rs]
            com.spanPtr[a], com.spans[a], com.revPtr[a], com.revSpans[a] = sp.ctypes.data, ss.ctypes.data, rp.ctypes.data, rs.ctypes.data
        com.ropeBuf = self.rope.ctypes.data
        pairs = np.array([(t, self.target[t]) for t in range(self.n) if self.target[t] >= 0], np.int32)
        self.states = np.zeros((self.depth + 1, self.n, self.dim), np.float32)
        self.ref_grad0 = np.zeros((self.n, self.dim), np.float32)
        self.ref_delta_embed = np.zeros((self.label_count, self.dim), np.float32)
        self.ref_delta_final = np.zeros((self.vocab, self.dim), np.float32)
        loss = o.lib.orc_model_step(C.byref(dims), self.depth, layers, C.byref(com), self.n, self.label_count, self.vocab, _ptr(self.label_ptr),
                                    _ptr(self.labels), _ptr(self.embed.deq), _ptr(self.final.deq), _ptr(self.bias), len(pairs), _ptr(pairs),
                                    _ptr(self.states), _ptr(self.ref_grad0), _ptr(self.ref_delta_embed), _ptr(self.ref_delta_final))
        self.ref_loss = loss
        return loss

    # ---- device side
    def device_model(self, k_tile=0, recompute=False, dither_seed=0):
        from tscale2_amd import lib as L
        m = L.Model(self.mode, self.dim, self.heads, self.ffn, self.lt, self.la, self.ls, len(self.att_width), self.vocab, self.label_count,
                    self.n, self.xp if self.experts else 0, self.experts, self.selected if self.experts else 0, k_tile, recompute, dither_seed)
        for d in range(self.depth):
            for i, q in enumerate(self.layers[d]):
                m.set_matrix(d, i, q.fast, q.scale)
        m.set_matrix(L.LAYER_EMBED, 0, self.embed.fast, self.embed.scale)
        m.set_matrix(L.LAYER_FINAL, 0, self.final.fast, self.final.scale)
        m.set_bias(self.bias)
        starts, finishes = [], []
        for sp, ss in self.spans:
            st = np.zeros(self.n, np.int32); fi = np.full(self.n, -1, np.int32)
            for t in range(self.n):
                if sp[t + 1] > sp[t]:
                    st[t], fi[t] = ss[sp[t]]
            starts.append(st); finishes.append(fi)
        m.set_batch(self.label_ptr, self.labels, self.target, starts, finishes, self.rope)
        return m


def scale_fit(got, ref):
    """least-squares scale of got on ref (1 = unbiased) and their correlation"""
    g = got.astype(np.float64).ravel(); r = ref.astype(np.float64).ravel()
    rr = (r * r).sum() + 1e-300
    return float((g * r).sum() / rr), float((g * r).sum() / (np.sqrt((g * g).sum() * rr) + 1e-300))


def rel_err(got, ref):
    d = got.astype(np.float64) - ref
    den = np.sqrt((ref.astype(np.float64) ** 2).mean()) + 1e-30
    return float(np.sqrt((d ** 2).mean()) / den), float(np.abs(d).max() / (np.abs(ref).max() + 1e-30))
