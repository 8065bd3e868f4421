"""Attention forward / backward on the GPU against the oracle (the reference's TAttentionComputer restated).
Inputs are bf16-representable so both sides see identical operands; the device rounds probabilities and score gradients to bf16
before the second product of each pair (fp32 accumulate), hence the tolerance: max |err| <= 1e-2 * max |ref| per tensor."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")
from golden_cases import causal_spans  # noqa: E402
from oracle_lib import Oracle  # noqa: E402


@pytest.fixture(scope="module")
def L():
    from tscale2_amd import lib
    lib.load()
    return lib


@pytest.fixture(scope="module")
def orc():
    return Oracle()


def bf16_round(a):
    return torch.from_numpy(a).bfloat16().float().numpy()


def spans_to_ranges(sp, spans, n, n_round):
    start = np.zeros(n_round, np.int32)
    finish = np.full(n_round, -1, np.int32)
    for t in range(n):
        assert sp[t + 1] - sp[t] <= 1
        if sp[t + 1] > sp[t]:
            start[t], finish[t] = spans[sp[t]]
    return start, finish


def ragged_spans(doc_lens, window):
    """documents of unequal length back to back: token t of a document that starts at d0 sees [max(d0, t - window), t - 1]"""
    n = int(sum(doc_lens))
    sp = np.zeros(n + 1, np.int32)
    spans = []
    t = 0
    for ln in doc_lens:
        d0 = t
        for _ in range(ln):
            a, b = max(d0, t - window), t - 1
            if b >= a:
                spans.append((a, b))
            sp[t + 1] = len(spans)
            t += 1
    return sp, np.array(spans, np.int32).reshape(-1, 2)


def run_case(L, orc, frag_count, frag_len, window, heads, slope, seed, grad_type, custom_spans=None):
    n = frag_count * frag_len
    sp, spans = causal_spans(frag_count, frag_len, window) if custom_spans is None else custom_spans
    if custom_spans is not None:
        n = sp.size - 1
    n_round = (n + 127) // 128 * 128
    r = np.random.default_rng(seed)
    # q, v are unit-rms heads and k ~ N(0,1) in the model; scaled so that logits have a realistic spread
    q = bf16_round(r.standard_normal((n, heads * 128)).astype(np.float32))
    k = bf16_round(r.standard_normal((n, heads * 128)).astype(np.float32))
    v = bf16_round(r.standard_normal((n, heads * 128)).astype(np.float32))
    dval = bf16_round(r.standard_normal((n, heads * 128)).astype(np.float32))
    ref = orc.attention(heads, 128, 128, slope, sp, spans, q, k, v, dval)
    att_dot_scale = float(np.float32(np.sqrt(np.float32(1.0 / 128))) * np.float32(0.5 / 0.693147))

    def padded(a):
        t = torch.zeros((n_round, a.shape[1]), dtype=torch.bfloat16, device="cuda")
        t[:n] = torch.from_numpy(a).cuda().bfloat16()
        return t
    tq, tk, tv, tdv = padded(q), padded(k), padded(v), padded(dval)
    start, finish = spans_to_ranges(sp, spans, n, n_round)
    ts, tf = torch.from_numpy(start).cuda(), torch.from_numpy(finish).cuda()
    val = torch.full((n_round, heads * 128), 7.0, dtype=torch.bfloat16, device="cuda")
    swl = torch.full((heads, n_round), -5.0, device="cuda")
    i16 = torch.int16
    L.att_forward(n, heads, tq.view(i16), tk.view(i16), tv.view(i16), ts, tf, att_dot_scale, slope, val.view(i16), swl)
    torch.cuda.synchronize()
    got_val = val.float().cpu().numpy()[:n]
    err = np.abs(got_val - ref["val"]).max() / np.abs(ref["val"]).max()
    print("valLookup rel err", err)
    assert err <= 1e-2
    want_l = ref["max_dp"] + np.log2(ref["sum_weight"])
    np.testing.assert_allclose(swl.cpu().numpy()[:, :n], want_l, rtol=1e-4, atol=1e-4)
    assert np.all(val.float().cpu().numpy()[n:] == 0) and np.all(swl.cpu().numpy()[:, n:] == 0)

    # backward uses the forward's statistics and the oracle's dScale (the device computes dScale in the gate kernel)
    ds = torch.zeros((heads, n_round), device="cuda")
    ds[:, :n] = torch.from_numpy(ref["dscale"]).cuda()
    rev_lo = torch.zeros(n_round // 128, dtype=torch.int32, device="cuda")
    rev_hi = torch.zeros(n_round // 128, dtype=torch.int32, device="cuda")
    L.call("ts2_att_build_rev", n, n_round, ts, tf, rev_lo, rev_hi)
    tdt = torch.float32 if grad_type == L.F32 else torch.bfloat16
    dq = torch.full((n_round, heads * 128), 3.0, dtype=tdt, device="cuda")
    dk = torch.full((n_round, heads * 128), 3.0, dtype=tdt, device="cuda")
    dv = torch.full((n_round, heads * 128), 3.0, dtype=tdt, device="cuda")
    vw = (lambda t: t) if grad_type == L.F32 else (lambda t: t.view(i16))
    L.att_backward(n, heads, tq.view(i16), tk.view(i16), tv.view(i16), tdv.view(i16), ts, tf, rev_lo, rev_hi, att_dot_scale, slope, swl, ds,
                   vw(dq), vw(dk), vw(dv), grad_type)
    torch.cuda.synchronize()
    for name, got in (("dq", dq), ("dk", dk), ("dv", dv)):
        g = got.float().cpu().numpy()
        err = np.abs(g[:n] - ref[name]).max() / np.abs(ref[name]).max()
        print(name, "rel err", err)
        assert err <= 1e-2, name
        assert np.all(g[n:] == 0), name
    # the same with the score gradients handed from the dK/dV kernel to the dQ kernel (5 products instead of 7): dK and dV are the very
    # same values, dQ is formed from dS rounded to bf16 where the other kernel rounds its own evaluation of it: equal to bf16 noise
    print("  ... dQ from the dK/dV kernel's score gradients", flush=True)
    ds_pair = L.att_ds_scratch(n_round, heads, ts, tf)
    ds_pair[1].fill_(0x7f)  # NaN patterns where nothing is written
    dq2, dk2, dv2 = torch.full_like(dq, 3.0), torch.full_like(dk, 3.0), torch.full_like(dv, 3.0)
    L.att_backward(n, heads, tq.view(i16), tk.view(i16), tv.view(i16), tdv.view(i16), ts, tf, rev_lo, rev_hi, att_dot_scale, slope, swl, ds,
                   vw(dq2), vw(dk2), vw(dv2), grad_type, ds=ds_pair)
    torch.cuda.synchronize()
    assert torch.equal(dk2, dk) and torch.equal(dv2, dv)
    g2 = dq2.float().cpu().numpy()
    err = np.abs(g2[:n] - ref["dq"]).max() / np.abs(ref["dq"]).max()
    print("dq (from dS) rel err", err, "against the other kernel", np.abs(g2 - dq.float().cpu().numpy()).max() / np.abs(ref["dq"]).max())
    assert err <= 1e-2 and np.all(g2[n:] == 0)
    assert np.abs(g2 - dq.float().cpu().numpy()).max() <= 4e-3 * np.abs(ref["dq"]).max()


def test_attention_window_and_slope(L, orc):
    print("case att window", flush=True)
    run_case(L, orc, frag_count=3, frag_len=100, window=64, heads=2, slope=0.5, seed=21, grad_type=L.F32)


def test_attention_full_causal_bf16_grads(L, orc):
    print("case att full causal", flush=True)
    run_case(L, orc, frag_count=2, frag_len=320, window=1024, heads=1, slope=0.0, seed=22, grad_type=L.BF16)


def test_attention_window_one(L, orc):
    print("case att window 1", flush=True)
    run_case(L, orc, frag_count=2, frag_len=70, window=1, heads=1, slope=0.0, seed=23, grad_type=L.F32)


def test_attention_remapped_block_order(L, orc):
    """a launch whose workgroup count is a multiple of 8 (the block order is then remapped per XCD), several 128-row blocks per
    sequence, a slope, key ranges that start inside a 64-row tile"""
    print("case att remapped order", flush=True)
    run_case(L, orc, frag_count=4, frag_len=256, window=200, heads=2, slope=0.25, seed=24, grad_type=L.BF16)


@pytest.mark.parametrize("window,slope,seed", [(96, 0.125, 31), (1000, 0.0, 32), (40, 0.0, 33)])
def test_attention_ragged_documents(L, orc, window, slope, seed):
    """documents of random lengths between 1 and 400 tokens: rows without a span (first tokens), 32-row blocks that straddle document
    starts (seen partly by one key block of a workgroup and completely by the other, so the dK/dV waves take their two-block and
    their one-block paths in turn and the hand-over counters run through both), windows that end inside a tile"""
    print("case att ragged documents", window, slope, flush=True)
    r = np.random.default_rng(seed)
    lens = []
    while sum(lens) < 1100:
        lens.append(int(r.integers(1, 400)))
    run_case(L, orc, 0, 0, window, heads=2, slope=slope, seed=seed, grad_type=L.BF16, custom_spans=ragged_spans(lens, window))


@pytest.mark.parametrize("slope", [0.0, 0.01])
def test_attention_one_sequence_of_2048_tokens(L, orc, slope):
    """the sequence length of config[3] (and twice config[2]'s): full causal spans over sixteen 128-row blocks, statistics accumulated
    over up to 2047 keys, the reverse ranges of the last blocks reaching back over the whole sequence, the position term at distance 2000"""
    print("case att 2048 tokens, slope", slope, flush=True)
    run_case(L, orc, frag_count=1, frag_len=2048, window=4096, heads=2, slope=slope, seed=25, grad_type=L.BF16)


def test_rope_and_head_norm_passes(L, orc):
    print("case rope/norm passes", flush=True)
    r = np.random.default_rng(24)
    n, n_round, heads = 150, 256, 2
    src = r.standard_normal((n, heads * 128)).astype(np.float32) * 0.3
    rope = orc.fill_rope_buf(128, n_round)
    want = orc.apply_rope(rope, 1.0, orc.normalize_state(src, heads))
    dst = torch.full((n_round, heads * 128), 5.0, dtype=torch.bfloat16, device="cuda")
    sc = torch.full((heads, n_round), -1.0, device="cuda")
    tr = torch.from_numpy(rope).cuda()
    L.call("ts2_row_tile_normalize_rope", n, n_round, torch.from_numpy(src).cuda(), L.F32, 1.0, 1, 1.0, tr, dst.view(torch.int16), sc)
    torch.cuda.synchronize()
    np.testing.assert_allclose(dst.float().cpu().numpy()[:n], want, rtol=2 ** -8, atol=2e-3)
    assert np.all(dst.float().cpu().numpy()[n:] == 0)
    rms = np.sqrt((src.reshape(n, heads, 128).astype(np.float64) ** 2).mean(-1))
    np.testing.assert_allclose(sc.cpu().numpy()[:, :n].T, rms, rtol=1e-5)
    # backward: oracle order = inverse rope, then norm backward against the un-rotated source
    g = r.standard_normal((n, heads * 128)).astype(np.float32)
    want_g = orc.normalize_state_backward(src, orc.apply_rope(rope, -1.0, g), heads)
    out = torch.zeros((n_round, heads * 128), device="cuda")
    L.call("ts2_backprop_row_tile_normalize_rope", n, n_round, torch.from_numpy(g).cuda(), L.F32, 1.0, dst.view(torch.int16), sc, tr, out, L.F32)
    torch.cuda.synchronize()
    # the stored normalised vector is bf16: 2^-8 relative on the source enters the projection
    assert np.abs(out.cpu().numpy()[:n] - want_g).max() <= 1e-2 * np.abs(want_g).max()


@pytest.mark.parametrize("with_norm,with_rope", [(True, True), (False, True), (True, False)])
def test_gradient_epilogue_with_eight_elements_per_lane_equals_the_four_wide_kernel(L, orc, with_norm, with_rope):
    """bf16 gradient -> e4m3 (the model's attention backward) takes the kernel with eight elements per lane; the same values given
    as fp32 take the four-wide kernel.  Same arithmetic except the order of the two tile sums: the e4m3 codes agree except for
    rare neighbours, pad rows are zero; 3 heads leave half-filled waves."""
    print("case gradient epilogue 8-wide", with_norm, with_rope, flush=True)
    r = np.random.default_rng(41)
    n, n_round, heads = 333, 384, 3
    g16 = torch.from_numpy(r.standard_normal((n, heads * 128)).astype(np.float32) * 4).bfloat16().cuda()
    sn = torch.from_numpy(r.standard_normal((n, heads * 128)).astype(np.float32)).bfloat16().cuda()
    sn[5, 128:256] = 0
    sc = (torch.rand((heads, n), device="cuda") + 0.5).contiguous()
    rope = torch.from_numpy(orc.fill_rope_buf(128, n_round)).cuda()
    a = torch.full((n_round, heads * 128), 9, dtype=torch.uint8, device="cuda")
    b = torch.full((n_round, heads * 128), 9, dtype=torch.uint8, device="cuda")
    args = (sn.view(torch.int16) if with_norm else None, sc if with_norm else None, rope if with_rope else None)
    L.call("ts2_backprop_row_tile_normalize_rope", n, n_round, g16.view(torch.int16), L.BF16, 0.75, *args, a, L.E4M3)
    L.call("ts2_backprop_row_tile_normalize_rope", n, n_round, g16.float().contiguous(), L.F32, 0.75, *args, b, L.E4M3)
    torch.cuda.synchronize()
    fa, fb = a.view(torch.float8_e4m3fn).float(), b.view(torch.float8_e4m3fn).float()
    assert (fa[n:] == 0).all() and (fb[n:] == 0).all()
    assert (a != b).float().mean().item() < 2e-3
    assert ((fa - fb).abs() <= fb.abs() * 2.0 ** -3 + 2.0 ** -9).all()
    if with_norm:
        assert (fa[5, 128:256] == 0).all()
