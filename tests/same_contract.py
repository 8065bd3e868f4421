"""Same-contract CPU model of the device step: the CPU oracle's arithmetic (its C primitives for attention, tile norm and the int8
quantisers; float64 numpy products) with a rounding at every point where the device stores a tensor in a narrower type - 8-bit norm
states and rg/vlg (i8 or e4m3), bf16 activations, fast gradients (bf16 or e4m3, power-of-two scaled), half logits, packed i8 deltas - and
the device's scale bookkeeping (1/24 storage units, gradMult / gradScale).  Where the fp32 oracle differs from the device by the 8-bit
storage noise (several per cent rms per delta), this model differs from it only by summation order, the hardware's 1-ulp exp / rcp /
sqrt and the rare roundings those flip: it is what the device results are compared with at <= 1e-2.

It follows the call order of the library's step driver (embedding, per layer normalise + FFN / attention forward, final layer and loss
gradient, backward loop with ScaleGrad / layer backward / normalisation backward, embedding delta), which is the order of the
reference's AddForward / AddBackward (src/gpt/compute/layer_ffn.cu:56-113, layer_att.cu:108-226, gpu_transformer.cu:260-471) with the
CPU path's factors.  Test infrastructure: FFN and attention layers in both 8-bit modes, MoE layers (layer_moe.cu:186-285) in e4m3 mode."""
import ctypes as C

import numpy as np

from model_harness import E4M3, I8, LT_ATT, LT_FFN, LT_MOE
from oracle_lib import _ptr

F32 = np.float32
VEC = F32(1 / 24)
DISCR = F32(1 / 32)
LN2F = F32(0.693147)


def dot(n):
    return F32(np.sqrt(F32(1.0) / F32(n)))


def bf16(x):
    """round to nearest even bfloat16, returned as fp32"""
    u = np.ascontiguousarray(x, F32).view(np.uint32)
    r = (u + np.uint32(0x7fff) + ((u >> np.uint32(16)) & np.uint32(1))) & np.uint32(0xffff0000)
    return r.view(F32)


_ORC = None


def e4m3(x):
    """round to nearest even OCP e4m3fn with saturation to +-448 (the device's conversion), returned as fp32"""
    global _ORC
    if _ORC is None:
        from oracle_lib import load_oracle
        _ORC = load_oracle()
    x = np.ascontiguousarray(x, F32)
    out = np.empty_like(x)
    _ORC.orc_round_e4m3_rne(_ptr(out), _ptr(x), C.c_long(x.size))
    return out


def e4m3_numpy(x):
    """the same rounding written independently in numpy (slow): quantum 2^(floor(log2 |x|) - 3), 2^-9 in the denormal range"""
    x = np.asarray(x, F32)
    a = np.minimum(np.abs(x.astype(np.float64)), 448.0)
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(np.where(a > 0, a, 1.0)))
    e = np.maximum(e, -6.0)
    q = np.exp2(e - 3)
    r = np.rint(a / q) * q
    return (np.sign(x) * np.minimum(r, 448.0)).astype(F32)


def i8(x):
    return np.clip(np.rint(np.asarray(x, F32)), -128, 127).astype(F32)


def f16(x):
    return np.asarray(x, F32).astype(np.float16).astype(F32)


def mm(a, b):
    """a [m][k] x b[n][k]^T in float64 (8-bit operands: every product is exact), rounded once to fp32"""
    return (a.astype(np.float64) @ b.astype(np.float64).T).astype(F32)


def lolu(g):
    g = g.astype(np.float64)
    m = 1 / (1 + np.exp(-2 * g))
    return np.where(g < -10, 0.0, m).astype(F32)


def tile_sum(x):
    n, d = x.shape
    return x.reshape(n, d // 128, 128).astype(np.float64).sum(-1)


def rep(t):
    return np.repeat(t, 128, axis=1)


def tile_norm_backprop(src, grad):
    """TileNormalizeBackprop per 128 tile: sqrt(128/sum2) * (grad - src * <src,grad>/sum2), zero for zero tiles"""
    s2 = tile_sum(src * src.astype(np.float64))
    dp = tile_sum(src.astype(np.float64) * grad)
    with np.errstate(divide="ignore", invalid="ignore"):
        sigma = np.where(s2 > 0, dp / s2, 0)
        scale = np.where(s2 > 0, np.sqrt(128 / s2), 0)
    return ((grad - src * rep(sigma)) * rep(scale)).astype(F32)


def rope(x, buf, direction):
    """rotate (even, odd) pairs of every 128-wide head by the row's (cos, sin) table [n][128]"""
    n, d = x.shape
    v = x.reshape(n, d // 128, 64, 2).astype(np.float64)
    c = buf.reshape(n, 1, 64, 2)[..., 0].astype(np.float64)
    s = buf.reshape(n, 1, 64, 2)[..., 1].astype(np.float64) * direction
    out = np.stack([v[..., 0] * c - v[..., 1] * s, v[..., 0] * s + v[..., 1] * c], -1)
    return out.reshape(n, d).astype(F32)


class SameContract:
    def __init__(self, h, k_tile=512):
        self.h, self.orc = h, h.orc
        self.mode = h.mode
        self.k_tile = k_tile if k_tile else 512
        self.q8 = i8 if h.mode == I8 else e4m3
        self.qfast = bf16 if h.mode == I8 else e4m3  # fast-gradient type
        self.n = h.n
        self.R = (h.n + max(self.k_tile, 128) - 1) // max(self.k_tile, 128) * max(self.k_tile, 128)
        tab = self.orc.e4m3_table(hw=True)
        self.val = (lambda m: m.fast.astype(F32)) if h.mode == I8 else (lambda m: tab[m.fast])
        self.acts, self.delta = {}, {}
        self.force = {}  # layer -> {"val16", "dq", "dk", "dv"}: tensors taken from the device instead of the model's own
        self.core = {}

    # ---- building blocks ---------------------------------------------------------------------------------------------------
    def normalize_state(self, state):
        """LayerNormalizeStateVecs: scale = rms(tile) / 24, norm = 8-bit(state / scale)"""
        s2 = tile_sum(state * state.astype(np.float64))
        discr = (np.sqrt(s2 / 128) * VEC).astype(F32)
        with np.errstate(divide="ignore", invalid="ignore"):
            inv = np.where(discr > 0, F32(1) / discr, 0).astype(F32)
        return self.q8(state * rep(inv)), discr

    def forward_mm(self, norm8, w, use_scale, alpha):
        return (mm(norm8, self.val(w)) * (F32(alpha) * (F32(w.scale) if use_scale else F32(1)))).astype(F32)

    def norm_rope(self, v, normalize, vec_scale, rope_buf):
        """the normalising / rotating store of a forward product: bf16(rope(v / (rms * vecScale))) and the tile scales"""
        discr = None
        if normalize:
            s2 = tile_sum(v * v.astype(np.float64))
            discr = (np.sqrt(s2 / 128) * F32(vec_scale)).astype(F32)
            with np.errstate(divide="ignore", invalid="ignore"):
                v = (v * rep(np.where(discr > 0, F32(1) / discr, 0).astype(F32))).astype(F32)
        if rope_buf is not None:
            v = rope(v, rope_buf, 1.0)
        return bf16(v), discr

    def backprop_dx(self, grad_fast, w, use_scale, alpha):
        """alpha [* scale] * grad * W: int8 quantises the gradient per row first (exact int32 sums, row scale in the epilogue)"""
        f = F32(alpha) * (F32(w.scale) if use_scale else F32(1))
        if self.mode == E4M3:
            return (mm(grad_fast, self.val(w).T) * f).astype(F32)
        n, gd = grad_fast.shape
        g = np.ascontiguousarray(grad_fast, F32)
        q = np.zeros((n, gd), np.int8); rs = np.zeros(n, F32)
        self.orc.lib.orc_quant_rowmax_i8(_ptr(g), _ptr(q), _ptr(rs), n, gd)
        acc = mm(q.astype(F32), self.val(w).T)
        return ((acc * rs[:, None]).astype(F32) * f).astype(F32)

    def backprop_delta(self, src8, grad_fast, grad_scale):
        """packed delta of grad^T src * (1/24) * gradScale, dequantised: int8 requantises the gradient per k-tile of rows"""
        n = src8.shape[0]
        if self.mode == E4M3:
            acc = mm(grad_fast.T, src8.T)
        else:
            R, kt = self.R, self.k_tile
            gd, sd = grad_fast.shape[1], src8.shape[1]
            g = np.zeros((R, gd), F32); g[:n] = grad_fast
            s = np.zeros((R, sd), np.int8); s[:n] = src8.astype(np.int8)
            qk = np.zeros((R, gd), np.int8); tsc = np.zeros(R // kt, F32)
            self.orc.lib.orc_quant_ktile_i8(_ptr(g), _ptr(qk), _ptr(tsc), R, gd, kt)
            acc = np.zeros((gd, sd), F32)
            self.orc.lib.orc_gemm_i8_nt_ktile(_ptr(np.ascontiguousarray(qk.T)), _ptr(np.ascontiguousarray(s.T)), _ptr(tsc), kt, C.c_float(1.0),
                                              _ptr(acc), gd, sd, R)
        return self.pack((acc * (VEC * F32(grad_scale))).astype(F32))

    def pack(self, v):
        """Compress to i8 + one scale per (row, 128-column tile), dequantised again"""
        v = np.ascontiguousarray(v, F32)
        rows, cols = v.shape
        q = np.zeros((rows, cols), np.int8); ts = np.zeros((cols // 128, rows), F32)
        self.orc.lib.orc_compress_delta(_ptr(v), _ptr(q), _ptr(ts), rows, cols)
        return q.astype(F32) * rep(np.ascontiguousarray(ts.T))

    # ---- layers ------------------------------------------------------------------------------------------------------------
    def ffn_forward(self, d, norm8):
        h = self.h
        W = h.layers[d]
        a = VEC * DISCR * dot(h.dim)
        wide16, wscale = self.norm_rope(self.forward_mm(norm8, W[0], True, a), True, VEC, None)
        gate16 = bf16(self.forward_mm(norm8, W[1], False, a))
        rg8 = self.q8(wide16 * lolu(gate16))
        self.acts[d] = (wide16, wscale, gate16, rg8)
        return self.forward_mm(rg8, W[2], True, VEC * DISCR * dot(h.ffn))

    def ffn_backward(self, d, norm8, sg_fast, grad_scale):
        h = self.h
        W = h.layers[d]
        wide16, wscale, gate16, rg8 = self.acts[d]
        drg = bf16(self.backprop_dx(sg_fast, W[2], True, DISCR * dot(h.ffn)))
        vv = (wide16 * VEC).astype(F32)
        mult = lolu(gate16)
        dgate = self.qfast(drg * vv * (mult * (1 - mult) * 2))
        src = (vv * rep((wscale / VEC).astype(F32))).astype(F32)
        dwide = self.qfast(tile_norm_backprop(src, (drg * mult).astype(F32)))
        a = DISCR * dot(h.dim)
        dnorm = (self.backprop_dx(dwide, W[0], True, a) + self.backprop_dx(dgate, W[1], False, a)).astype(F32)
        self.delta[d] = [self.backprop_delta(norm8, dwide, grad_scale), self.backprop_delta(norm8, dgate, grad_scale),
                         self.backprop_delta(rg8, sg_fast, grad_scale)]
        return dnorm

    def att_forward(self, d, norm8):
        h = self.h
        W = h.layers[d]
        a = VEC * DISCR * dot(h.dim)
        q16, qscale = self.norm_rope(self.forward_mm(norm8, W[0], True, a), True, 1.0, h.rope)
        k16, _ = self.norm_rope(self.forward_mm(norm8, W[1], True, a), False, 1.0, h.rope)
        v16, vscale = self.norm_rope(self.forward_mm(norm8, W[2], True, a), True, 1.0, None)
        gate16 = bf16(self.forward_mm(norm8, W[3], False, a))
        sp, ss = h.spans[int(h.la[d])]
        ss = np.ascontiguousarray(ss) if len(ss) else np.zeros((1, 2), np.int32)
        H = h.heads
        val = np.zeros((self.n, H * 128), F32); sw = np.zeros((H, self.n), F32); mx = np.zeros((H, self.n), F32)
        self.orc.lib.orc_attention_forward(self.n, H, 128, 128, C.c_float(float(h.ls[d])), C.c_float(1.0), _ptr(sp), _ptr(ss), _ptr(q16), _ptr(k16),
                                           _ptr(v16), _ptr(val), _ptr(sw), _ptr(mx))
        val16 = bf16(val)
        self.core = {"val16": val16}
        if d in self.force and "val16" in self.force[d]:
            val16 = self.force[d]["val16"]  # continue from the device's own attention output
        vlg8 = self.q8(val16 * lolu(gate16) * F32(24))
        self.acts[d] = (q16, qscale, k16, v16, vscale, gate16, val16, vlg8, sw, mx)
        return self.forward_mm(vlg8, W[4], True, VEC * DISCR * dot(H * 128))

    def att_backward(self, d, norm8, sg_fast, grad_scale):
        h = self.h
        W = h.layers[d]
        H = h.heads
        q16, qscale, k16, v16, vscale, gate16, val16, vlg8, sw, mx = self.acts[d]
        dvlg = bf16(self.backprop_dx(sg_fast, W[4], True, DISCR * dot(H * 128)))
        delta_comb = self.backprop_delta(vlg8, sg_fast, grad_scale)
        mult = lolu(gate16)
        dgate = self.qfast(dvlg * val16 * (mult * (1 - mult) * 2))
        dval = (dvlg * mult).astype(F32)
        dscale = np.ascontiguousarray(tile_sum(val16.astype(np.float64) * dval).T.astype(F32))  # [head][row]
        dval16 = bf16(dval)
        sp, ss = h.spans[int(h.la[d])]
        rp, rs = h.rev[int(h.la[d])]
        ss = np.ascontiguousarray(ss) if len(ss) else np.zeros((1, 2), np.int32)
        rs = np.ascontiguousarray(rs) if len(rs) else np.zeros((1, 2), np.int32)
        dq = np.zeros_like(q16); dk = np.zeros_like(q16); dv = np.zeros_like(q16)
        sl, am = C.c_float(float(h.ls[d])), C.c_float(1.0)
        L = self.orc.lib
        L.orc_attention_grad_q(self.n, H, 128, 128, sl, am, _ptr(sp), _ptr(ss), _ptr(q16), _ptr(k16), _ptr(v16), _ptr(dval16), _ptr(dscale), _ptr(sw),
                               _ptr(mx), _ptr(dq))
        L.orc_attention_grad_k(self.n, H, 128, 128, sl, am, _ptr(rp), _ptr(rs), _ptr(q16), _ptr(k16), _ptr(v16), _ptr(dval16), _ptr(dscale), _ptr(sw),
                               _ptr(mx), _ptr(dk), _ptr(dv))
        dq, dk, dv = bf16(dq), bf16(dk), bf16(dv)
        self.core.update(dq=dq, dk=dk, dv=dv, dval16=dval16, dscale=dscale, dgate=dgate)
        if d in self.force and "dq" in self.force[d]:
            dq, dk, dv = self.force[d]["dq"], self.force[d]["dk"], self.force[d]["dv"]  # ... and from its attention gradients
        # epilogues: norm backward against the stored rotated vector times its scale, then the inverse rotation
        dqf = self.qfast(rope(tile_norm_backprop((q16 * rep(np.ascontiguousarray(qscale))).astype(F32), dq), h.rope, -1.0))
        dkf = self.qfast(rope(dk, h.rope, -1.0))
        dvf = self.qfast(tile_norm_backprop((v16 * rep(np.ascontiguousarray(vscale))).astype(F32), dv))
        a = DISCR * dot(h.dim)
        dnorm = (self.backprop_dx(dqf, W[0], True, a) + self.backprop_dx(dkf, W[1], True, a) + self.backprop_dx(dvf, W[2], True, a) +
                 self.backprop_dx(dgate, W[3], False, a)).astype(F32)
        self.delta[d] = [self.backprop_delta(norm8, g, grad_scale) for g in (dqf, dkf, dvf, dgate)] + [delta_comb]
        return dnorm

    # ---- MoE layer: every (token, slot) pair is a row of its expert; the device groups those rows by expert, this model loops over experts
    def moe_route(self, sel):
        """MoeCalcSampleExpertLists: top-k by value with first-index ties, w = exp((s - max) / 2), scaled so that sum w^2 = experts"""
        n, E = sel.shape
        K = self.h.selected
        v = sel.astype(F32).copy()
        ids = np.zeros((n, K), np.int64); w = np.zeros((n, K), F32)
        rows = np.arange(n)
        for z in range(K):
            ids[:, z] = np.argmax(v, 1)  # first index among equals
            top = v[rows, ids[:, z]]
            if z == 0:
                mx = top.copy()
            w[:, z] = np.exp(((top - mx) * F32(0.5)).astype(F32)).astype(F32)
            v[rows, ids[:, z]] = F32(-1e10)
        scale = (np.sqrt(F32(E)) * np.sqrt(F32(1) / (w * w).sum(1, dtype=F32))).astype(F32)
        return ids, (w * scale[:, None]).astype(F32)

    def moe_forward(self, d, norm8):
        h = self.h
        assert self.mode == E4M3
        W = h.layers[d]
        E, K, X, D, n = h.experts, h.selected, h.xp, h.dim, self.n
        a = VEC * DISCR * dot(D)
        sel = self.forward_mm(norm8, W[3], False, a)
        ids, wts = self.moe_route(sel)
        we, wg, wc = self.val(W[0]).reshape(E, X, D), self.val(W[1]).reshape(E, X, D), self.val(W[2]).reshape(E, D, X)
        wide16 = np.zeros((n, K, X), F32); wscale = np.zeros((n, K, X // 128), F32); gate16 = np.zeros((n, K, X), F32)
        rg8 = np.zeros((n, K, X), F32); contract = np.zeros((n, K, D), F32)
        for k in range(K):
            for e in range(E):
                r = np.nonzero(ids[:, k] == e)[0]
                if not len(r):
                    continue
                raw = (mm(norm8[r], we[e]) * (a * F32(W[0].scale))).astype(F32)
                wide16[r, k], wscale[r, k] = self.norm_rope(raw, True, VEC, None)
                gate16[r, k] = bf16((mm(norm8[r], wg[e]) * a).astype(F32))
                rg8[r, k] = self.q8((wide16[r, k] * lolu(gate16[r, k])).astype(F32) * wts[r, k][:, None])
                contract[r, k] = bf16((mm(rg8[r, k], wc[e]) * (VEC * DISCR * dot(E * X) * F32(W[2].scale))).astype(F32))
        self.acts[d] = (ids, wts, wide16, wscale, gate16, rg8)
        out = contract[:, 0]
        for k in range(1, K):
            out = (out + contract[:, k]).astype(F32)
        return out

    def moe_backward(self, d, norm8, sg_fast, grad_scale):
        h = self.h
        W = h.layers[d]
        E, K, X, D, n = h.experts, h.selected, h.xp, h.dim, self.n
        ids, wts, wide16, wscale, gate16, rg8 = self.acts[d]
        we, wg, wc = self.val(W[0]).reshape(E, X, D), self.val(W[1]).reshape(E, X, D), self.val(W[2]).reshape(E, D, X)
        dwide = np.zeros((n, K, X), F32); dgate = np.zeros((n, K, X), F32); gm = np.zeros((n, K), F32)
        full = np.zeros((n, K, D), F32)
        f2 = DISCR * dot(E * X) * F32(W[2].scale)
        f0 = DISCR * dot(D)
        deltas = [np.zeros(W[i].fast.shape, F32) for i in range(3)]
        for k in range(K):
            for e in range(E):
                r = np.nonzero(ids[:, k] == e)[0]
                if not len(r):
                    continue
                drg = bf16((mm(sg_fast[r], wc[e].T) * f2).astype(F32))
                vv = (wide16[r, k] * VEC).astype(F32)
                mult = lolu(gate16[r, k])
                moe = wts[r, k][:, None]
                gm[r, k] = (drg.astype(np.float64) * vv * mult).sum(1).astype(F32)
                dgate[r, k] = self.qfast((drg * vv * (mult * (1 - mult) * 2)).astype(F32) * moe)
                src = (vv * rep((wscale[r, k] / VEC).astype(F32))).astype(F32)
                dwide[r, k] = self.qfast(tile_norm_backprop(src, ((drg * mult).astype(F32) * moe).astype(F32)))
                # expand and gate products in one launch: the sums of the first are rescaled to the second's factor, one multiply at the end
                full[r, k] = bf16(((mm(dwide[r, k], we[e].T).astype(np.float64) * float(f0 * F32(W[0].scale)) +
                                    mm(dgate[r, k], wg[e].T).astype(np.float64) * float(f0))).astype(F32))
        # the deltas of an expert contract over all its rows, whatever their slot
        for e in range(E):
            tk = np.nonzero(ids == e)
            if not len(tk[0]):
                continue
            src = norm8[tk[0]]
            g = F32(VEC * F32(grad_scale))
            deltas[2][e * D:(e + 1) * D] = (mm(sg_fast[tk[0]].T, rg8[tk].T) * g).astype(F32)
            deltas[0][e * X:(e + 1) * X] = (mm(dwide[tk].T, src.T) * g).astype(F32)
            deltas[1][e * X:(e + 1) * X] = (mm(dgate[tk].T, src.T) * g).astype(F32)
        # BackpropMoe (CpuBackpropMoe restricted to the selected experts)
        ms = np.sqrt(F32(E))
        w = (wts / ms).astype(F32); g = (gm * ms).astype(F32)
        avrg = (w * g).sum(1, dtype=F32)[:, None]
        dsel = np.zeros((n, E), F32)
        dsel[np.arange(n)[:, None], ids] = self.qfast(((w * g - w * w * avrg) * F32(0.5)).astype(F32))
        dnorm = full[:, 0]
        for k in range(1, K):
            dnorm = (dnorm + full[:, k]).astype(F32)
        dnorm = (dnorm + self.backprop_dx(dsel, W[3], False, f0)).astype(F32)
        self.core = {"dsel": dsel, "ids": ids, "wts": wts}
        self.delta[d] = [self.pack(deltas[0]), self.pack(deltas[1]), self.pack(deltas[2]), self.backprop_delta(norm8, dsel, grad_scale)]
        return dnorm

    # ---- one layer / the final layer on given inputs -------------------------------------------------------------------------------
    def layer_forward(self, d, norm8):
        """the layer's addition to the residual state from its 8-bit input"""
        lt = int(self.h.lt[d])
        return self.ffn_forward(d, norm8) if lt == LT_FFN else self.moe_forward(d, norm8) if lt == LT_MOE else self.att_forward(d, norm8)

    def layer_backward(self, d, norm8, scale, grad):
        """one step of the backward loop: ScaleGrad, the layer's backward (deltas to self.delta[d]), the normalisation backward with the
        residual add.  norm8 / scale: the layer's stored input and its tile scales; grad: the fp32 state gradient coming in."""
        gm = F32(self.orc.lib.orc_grad_mult(float(np.abs(grad).max())))
        gs = F32(1) / gm
        sg_fast = self.qfast(grad * gm)
        lt = int(self.h.lt[d])
        back = self.ffn_backward if lt == LT_FFN else self.moe_backward if lt == LT_MOE else self.att_backward
        dn = back(d, norm8, sg_fast, gs)
        return (tile_norm_backprop((norm8 * rep(scale)).astype(F32), (dn * gs).astype(F32)) + grad).astype(F32)

    def final_backward(self, fn8, scale):
        """final layer: half logits, base-2 soft-max with the maximum not below 0, (onehot - p) in bf16, bf16 products"""
        h = self.h
        D = h.dim
        logits = f16(self.forward_mm(fn8, h.final, True, VEC * DISCR * dot(D) / LN2F))
        z = logits.astype(np.float64) + h.bias.astype(np.float64)
        m = np.maximum(z.max(1), 0)
        w = np.exp2(z - m[:, None])
        p = w / w.sum(1, keepdims=True)
        live = h.target >= 0
        onehot = np.zeros_like(p)
        onehot[np.nonzero(live)[0], h.target[live]] = 1
        self.grad_v = bf16(np.where(live[:, None], onehot - p, 0).astype(F32))
        self.loss = float(np.log(p[np.nonzero(live)[0], h.target[live]]).sum() / live.sum())
        wf = self.val(h.final)
        dnorm = (mm(self.grad_v, wf.T) * (DISCR * dot(D) * F32(h.final.scale))).astype(F32)
        self.delta_final = self.pack((mm(self.grad_v.T, fn8.T) * VEC).astype(F32))
        return tile_norm_backprop((fn8 * rep(scale)).astype(F32), dnorm)

    def embedding_delta(self, grad):
        h = self.h
        de = np.zeros((h.label_count, h.dim), np.float64)
        for t in range(self.n):
            for k in range(h.label_ptr[t], h.label_ptr[t + 1]):
                lab = int(h.labels[k])
                de[lab & 0x7fffffff] += grad[t] * (-1 if lab & 0x80000000 else 1)
        return de.astype(F32)

    # ---- step --------------------------------------------------------------------------------------------------------------
    def run(self):
        h = self.h
        n, D = self.n, h.dim
        depth = h.depth
        self.acts, self.delta = {}, {}
        emb = self.val(h.embed)
        state = np.zeros((n, D), F32)
        s = DISCR * F32(h.embed.scale)
        for t in range(n):
            for k in range(h.label_ptr[t], h.label_ptr[t + 1]):
                lab = int(h.labels[k])
                state[t] += emb[lab & 0x7fffffff] * (-s if lab & 0x80000000 else s)
        norm, scale = [None] * (depth + 1), [None] * (depth + 1)
        norm[0], scale[0] = self.normalize_state(state)
        for d in range(depth):
            state = (state + self.layer_forward(d, norm[d])).astype(F32)
            norm[d + 1], scale[d + 1] = self.normalize_state(state)
        self.state = state
        grad = self.final_backward(norm[depth], scale[depth])
        for d in range(depth - 1, -1, -1):
            grad = self.layer_backward(d, norm[d], scale[d], grad)
        self.state_grad = grad
        self.delta_embed = self.embedding_delta(grad)
        return self
