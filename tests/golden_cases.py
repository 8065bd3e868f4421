"""Seeded cases shared by the fixture generator (run against the reference's own code) and the oracle tests."""
import numpy as np

F32 = np.float32


def _rng(seed):
    return np.random.default_rng(seed)


def case_linalg(o):
    r = _rng(101)
    vec = r.standard_normal((37, 96)).astype(F32)
    kqv = (r.standard_normal((40, 96)) * 0.3).astype(F32)
    rg = r.standard_normal((37, 40)).astype(F32)
    g0 = r.standard_normal((37, 96)).astype(F32)
    return {"fwd": o.mul_forward(vec, kqv), "bwd": o.mul_backward_accum(g0, kqv, rg), "delta": o.sum_rank_one(vec, rg)}


def case_norm_lolu(o):
    r = _rng(102)
    s = r.standard_normal((19, 256)).astype(F32)
    s[3, 128:] = 0  # an all-zero tile
    d = r.standard_normal((19, 256)).astype(F32)
    gate = (r.standard_normal((19, 256)) * 6).astype(F32)  # reaches the +-20 clamps (2*gate)
    gg, gv = o.backprop_lolu(gate, s, d)
    return {"norm": o.normalize_state(s, 2), "norm_bwd": o.normalize_state_backward(s, d, 2), "norm4": o.normalize_state(s, 4),
            "lolu": o.lolu(gate, s), "dgate": gg, "dvals": gv}


def case_rope(o):
    r = _rng(103)
    buf = o.fill_rope_buf(128, 70)
    p = r.standard_normal((70, 256)).astype(F32)
    fwd = o.apply_rope(buf, 1.0, p)
    return {"buf": buf, "fwd": fwd, "back": o.apply_rope(buf, -1.0, fwd)}


def att_inputs(seed, n, heads, qdim, ttdim):
    r = _rng(seed)
    q = r.standard_normal((n, heads * qdim)).astype(F32)
    k = r.standard_normal((n, heads * qdim)).astype(F32)
    v = r.standard_normal((n, heads * ttdim)).astype(F32)
    dv = r.standard_normal((n, heads * ttdim)).astype(F32)
    return q, k, v, dv


def causal_spans(frag_count, frag_len, window):
    sp = [0]
    spans = []
    for f in range(frag_count):
        p = f * frag_len
        for t in range(frag_len):
            a, b = max(0, t - window), t - 1
            if b >= a:
                spans.append((a + p, b + p))
            sp.append(len(spans))
    return np.array(sp, np.int32), np.array(spans, np.int32).reshape(-1, 2)


def case_attention(o):
    out = {}
    # two fragments of 24 rows, window 7, slope 0.5, 2 heads of 32
    sp, spans = causal_spans(2, 24, 7)
    q, k, v, dv = att_inputs(104, 48, 2, 32, 32)
    res = o.attention(2, 32, 32, 0.5, sp, spans, q, k, v, dv)
    out.update({"a_" + n: a for n, a in res.items()})
    # full causal window, slope 0, head dim 128, with an irregular extra span on one row
    sp2, spans2 = causal_spans(1, 20, 64)
    q, k, v, dv = att_inputs(105, 20, 1, 128, 128)
    res = o.attention(1, 128, 128, 0.0, sp2, spans2, q * 0.3, k * 0.3, v, dv)
    out.update({"b_" + n: a for n, a in res.items()})
    rp, rs = o.transpose_attention(sp, spans)
    out["rev_ptr"] = rp
    out["rev_spans"] = rs
    return out


def case_convert(o):
    r = _rng(106)
    x = np.concatenate([r.standard_normal(4096) * 40, np.linspace(-200, 200, 2048), np.arange(-130, 126) + 0.5,
                        np.array([3e9, -3e9, 2.5, 3.5, -2.5, 0.0] + [0.0] * 26)]).astype(F32)
    x = x[: (x.size // 32) * 32]
    tab = o.e4m3_table()
    # every e4m3 grid point, every midpoint between neighbours and random values over the whole range incl. under/overflow
    pos = np.sort(np.unique(np.abs(tab)))
    mids = (pos[1:] + pos[:-1]) / 2
    y = np.concatenate([pos, -pos, mids, -mids, np.nextafter(mids, F32(1e9)), np.nextafter(mids, F32(0)),
                        r.standard_normal(4096) * 3, r.standard_normal(512) * 300, r.standard_normal(512) * 0.004,
                        np.array([1e-8, 500, 1e6, -1e6], F32)]).astype(F32)
    y = y[: (y.size // 8) * 8]
    return {"i8": o.convert_i8(x, 1.0), "i8s": o.convert_i8(x, 0.37), "e4": o.convert_e4m3(y, 1.0), "e4s": o.convert_e4m3(y, 7.3), "tab": tab}


MODEL_STRINGS = ["e256h2d4ffn8w64", "e2048h16d12ffn64w1024", "e512h4d1ffn16w256", "e1024xp512moe64moes2h8d1w128", "e512xp256moe8moes2h4d26w512"]


def case_model_schedule(o):
    """layer schedule of a model string (InitAlibi, src/gpt/model_params/model_dim.cpp:82-158): the oracle builds it from the numbers
    the test harness reads out of the string; the reference build parses the string itself and also reports those numbers"""
    from model_harness import parse_model_descr
    out = {}
    for i, descr in enumerate(MODEL_STRINGS):
        dims, wide = parse_model_descr(descr)
        r = o.model_schedule(descr, int(dims[9]), int(dims[6]), wide)
        out[f"{i}_dims"] = r.get("dims", dims)
        for k in ("layer_type", "layer_att_id", "layer_slope", "att_width"):
            out[f"{i}_{k}"] = r[k]
    return out


def case_label_data(o):
    """nodes of a batch (InitLabelData with noise labels disabled, src/gpt/att/sliding_window.cpp:269-306): labels, targets and the
    causal spans of every attention type, as the test harness builds them"""
    from model_harness import make_batch, parse_model_descr
    out = {}
    for i, (descr, vocab, fc, fl) in enumerate([("e256h2d4ffn8w64", 256, 3, 70), ("e256h2d1ffn8w16", 50, 2, 40), ("e256h2d4ffn8w1024", 1000, 2, 150)]):
        tokens = _rng(200 + i).integers(0, vocab, (fc, fl)).astype(np.int32)
        dims, wide = parse_model_descr(descr)
        widths = o.model_schedule(descr, int(dims[9]), int(dims[6]), wide)["att_width"]
        if o.use_ref:
            tg = np.full((fc, fl), -1, np.int32)
            tg[:, :-1] = tokens[:, 1:]
            for a in range(len(widths)):
                r = o.ref_label_data(descr, vocab, tokens, tg, a)
                for k in ("label_count", "label_ptr", "labels", "target_pairs"):
                    out[f"{i}_{k}"] = r[k]
                out[f"{i}_span_ptr{a}"] = r["span_ptr"]
                out[f"{i}_spans{a}"] = r["spans"].reshape(-1, 2)
        else:
            b = make_batch(o, vocab, tokens, widths)
            out[f"{i}_label_count"] = np.array([b["label_count"]], np.int32)
            out[f"{i}_label_ptr"] = b["label_ptr"]
            out[f"{i}_labels"] = b["labels"]
            rows = np.nonzero(b["target"] >= 0)[0]
            out[f"{i}_target_pairs"] = np.stack([rows, b["target"][rows]], 1).astype(np.int32)
            for a, (sp, ss) in enumerate(b["spans"]):
                out[f"{i}_span_ptr{a}"] = sp
                out[f"{i}_spans{a}"] = np.asarray(ss, np.int32).reshape(-1, 2)
    return out


def build_cases():
    return {"linalg": case_linalg, "norm_lolu": case_norm_lolu, "rope": case_rope, "attention": case_attention, "convert": case_convert,
            "model_schedule": case_model_schedule, "label_data": case_label_data}
