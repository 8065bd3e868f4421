"""Direct parity of the MoE gradient-movement kernels through the C ABI, at the MoE benchmark's shape (64 experts, top-2, expert
width 512 = four norm tiles per expert slab):
  ts2_moe_group_samples / ts2_combine_experts   against numpy gather / gather-sum (bit-exact)
  ts2_backprop_moe                               against CpuBackpropMoe restated (oracle/moe.c, layer_moe.cu:330-358)
  ts2_backprop_row_tile_normalize_lolu_moe       against BackpropScaleExperts + BackpropLoLU + NormalizeStateBackward of the CPU layer
                                                 (layer_moe.cu:379-403,488-537; cpu_util.cpp:100-186)"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")
from oracle_lib import Oracle, _ptr  # noqa: E402

NAMES = ("ids", "w", "off", "eo", "tile", "sid", "sw", "bc")
VEC = np.float32(1 / 24)


class Tables(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in NAMES]


def route(L, len_, experts, selected, seed):
    r = np.random.default_rng(seed)
    sel = r.standard_normal((len_, experts)).astype(np.float32)
    total = len_ * selected
    len_moe = (total + 128 * experts + 127) // 128 * 128
    dev = "cuda"
    t = {"ids": torch.zeros(total, dtype=torch.int32, device=dev), "w": torch.zeros(total, device=dev),
         "off": torch.zeros(total, dtype=torch.int32, device=dev), "eo": torch.zeros(experts + 2, dtype=torch.int32, device=dev),
         "tile": torch.zeros(len_moe // 128, dtype=torch.int32, device=dev), "sid": torch.zeros(len_moe, dtype=torch.int32, device=dev),
         "sw": torch.zeros(len_moe, device=dev), "bc": torch.zeros(((total + 255) // 256) * experts, dtype=torch.int32, device=dev)}
    tb = Tables(*[t[n].data_ptr() for n in NAMES])
    L.call("ts2_moe_route", len_, len_moe, experts, selected, torch.from_numpy(sel).cuda(), L.F32, C.byref(tb))
    torch.cuda.synchronize()
    host = {n: t[n].cpu().numpy() for n in NAMES[:-1]}
    # grouped row of every (token, slot)
    host["row"] = (host["eo"][host["ids"]] + host["off"]).reshape(len_, selected)
    return sel, t, tb, len_moe, host


@pytest.fixture(scope="module")
def lib():
    from tscale2_amd import lib as L
    L.load()
    return L


@pytest.mark.parametrize("elem", [1, 2])
def test_group_samples_is_the_row_gather(lib, elem):
    L = lib
    len_, E, K, dim = 3000, 64, 2, 1024
    print("case moe group samples", elem, flush=True)
    _, t, tb, len_moe, host = route(L, len_, E, K, 21)
    r = np.random.default_rng(22)
    dt = np.uint8 if elem == 1 else np.uint16
    src = r.integers(0, 255 if elem == 1 else 65535, (len_, dim)).astype(dt)
    tdt = torch.uint8 if elem == 1 else torch.int16
    dst = torch.full((len_moe, dim), 77, dtype=tdt, device="cuda")
    L.call("ts2_moe_group_samples", len_moe, elem, torch.from_numpy(src.view(np.uint8 if elem == 1 else np.int16)).cuda(), t["sid"], dst)
    torch.cuda.synchronize()
    got = dst.cpu().numpy().view(dt)
    sid = host["sid"]
    want = np.where(sid[:, None] >= 0, src[np.maximum(sid, 0)], 0).astype(dt)
    assert np.array_equal(got, want)
    assert (sid >= 0).sum() == len_ * K


@pytest.mark.parametrize("src_type", ["f32", "bf16"])
def test_combine_experts_is_the_gather_sum_in_slot_order(lib, src_type):
    L = lib
    len_, E, K, dim = 3000, 64, 2, 1024
    print("case moe combine", src_type, flush=True)
    _, t, tb, len_moe, host = route(L, len_, E, K, 23)
    r = np.random.default_rng(24)
    src = torch.from_numpy(r.standard_normal((len_moe, dim)).astype(np.float32)).cuda()
    if src_type == "bf16":
        src = src.bfloat16()
    srcf = src.float().cpu().numpy()
    res0 = r.standard_normal((len_, dim)).astype(np.float32)
    alpha = np.float32(0.37)
    ap = torch.tensor([1.5], device="cuda")
    s = alpha * np.float32(1.5)
    ty = L.F32 if src_type == "f32" else L.BF16
    for add in (0, 1):
        res = torch.from_numpy(res0.copy()).cuda()
        L.call("ts2_combine_experts", len_, K, src, ty, C.byref(tb), float(alpha), ap, res, add)
        torch.cuda.synchronize()
        want = np.zeros((len_, dim), np.float32)
        for k in range(K):
            want = want + srcf[host["row"][:, k]]
        want = want * s
        if add:
            want = want + res0
        assert np.array_equal(res.cpu().numpy(), want), add


def test_backprop_moe_matches_cpu_backprop_moe(lib):
    L = lib
    orc = Oracle()
    len_, E, K = 3000, 64, 2
    print("case moe routing backward", flush=True)
    sel, t, tb, len_moe, host = route(L, len_, E, K, 25)
    r = np.random.default_rng(26)
    dxw = r.standard_normal(len_moe).astype(np.float32)
    len_round = (len_ + 127) // 128 * 128
    ids = host["ids"].reshape(len_, K); w = host["w"].reshape(len_, K)
    moe = np.zeros((len_, E), np.float32); dmoe = np.zeros((len_, E), np.float32)
    for k in range(K):
        moe[np.arange(len_), ids[:, k]] = w[:, k]
        dmoe[np.arange(len_), ids[:, k]] = dxw[host["row"][:, k]]
    orc.lib.orc_cpu_backprop_moe(len_, E, _ptr(moe), _ptr(dmoe))
    for ty, tdt, tol in ((L.F32, torch.float32, 2e-6), (L.BF16, torch.bfloat16, 4e-3)):
        out = torch.full((len_round, 128), 9, dtype=tdt, device="cuda")  # 128 columns: the select matrix is padded to a tile
        L.call("ts2_backprop_moe", len_, len_round, E, K, C.byref(tb), torch.from_numpy(dxw).cuda(), out, ty)
        torch.cuda.synchronize()
        got = out.float().cpu().numpy()
        assert (got[:, E:] == 0).all() and (got[len_:] == 0).all()
        np.testing.assert_allclose(got[:len_, :E], dmoe, rtol=tol, atol=tol * np.abs(dmoe).max())


@pytest.mark.parametrize("grad_type", ["f32", "bf16"])
def test_gate_and_norm_backward_over_grouped_rows_matches_the_cpu_layer(lib, grad_type):
    """64 experts of width 512 (four norm tiles per slab): per grouped row the CPU layer computes, for the row's token and expert slab,
    gradMoe = <LoLU(gate, wn), drg>, drg *= moe, (dgate, dwn) = BackpropLoLU, dwide = NormalizeStateBackward(wide, dwn)"""
    L = lib
    orc = Oracle()
    len_, E, K, X = 700, 64, 2, 512
    print("case moe gate/norm backward", grad_type, flush=True)
    _, t, tb, len_moe, host = route(L, len_, E, K, 27)
    r = np.random.default_rng(28)
    tiles = X // 128
    # device inputs over grouped rows: gate and the normalised wide (1/24 units) in bf16, the tile scales, the gradient of rg
    wide = (r.standard_normal((len_moe, X)) * np.exp(r.standard_normal((len_moe, 1)))).astype(np.float32)
    wide[5, 128:256] = 0  # a zero tile
    rms = np.sqrt((wide.reshape(len_moe, tiles, 128).astype(np.float64) ** 2).mean(-1)).astype(np.float32)
    tsc = (rms * VEC).astype(np.float32)                                         # [row][tile]
    with np.errstate(divide="ignore", invalid="ignore"):
        vals = np.where(np.repeat(tsc, 128, 1) > 0, wide / np.repeat(tsc, 128, 1), 0).astype(np.float32)
    vals16 = torch.from_numpy(vals).cuda().bfloat16()
    gate16 = torch.from_numpy((r.standard_normal((len_moe, X)) * 1.5).astype(np.float32)).cuda().bfloat16()
    grad = torch.from_numpy(r.standard_normal((len_moe, X)).astype(np.float32)).cuda()
    if grad_type == "bf16":
        grad = grad.bfloat16()
    tsc_dev = torch.from_numpy(np.ascontiguousarray(tsc.T)).cuda()                 # [tile][row]
    d_gate = torch.full((len_moe, X), 9, dtype=torch.bfloat16, device="cuda"); d_vals = torch.full_like(d_gate, 9)
    dxw = torch.full((len_moe,), 9.0, device="cuda")
    L.call("ts2_backprop_row_tile_normalize_lolu_moe", len_moe, t["sw"], gate16, vals16, float(VEC), tsc_dev, grad,
           L.F32 if grad_type == "f32" else L.BF16, 1.0, d_gate, d_vals, L.BF16, dxw)
    torch.cuda.synchronize()
    # CPU side on exactly the values the device reads: wn = vals16 / 24, wide = wn * (tile scale / (1/24))
    wn = (vals16.float().cpu().numpy() * VEC).astype(np.float32)
    widec = (wn * np.repeat(tsc / VEC, 128, 1).astype(np.float32)).astype(np.float32)
    gatec = gate16.float().cpu().numpy()
    drg = grad.float().cpu().numpy().copy()
    moe = host["sw"].reshape(len_moe, 1).astype(np.float32)                        # one "expert" per grouped row: its routing weight
    rg = np.zeros_like(wn)
    orc.lib.orc_lolu(_ptr(gatec), _ptr(wn), _ptr(rg), len_moe, X)
    grad_moe = np.zeros((len_moe, 1), np.float32)
    orc.lib.orc_backprop_scale_experts(len_moe, 1, X, _ptr(moe), _ptr(rg), _ptr(grad_moe), _ptr(drg))
    want_gate = np.zeros_like(wn); dwn = np.zeros_like(wn); want_vals = np.zeros_like(wn)
    orc.lib.orc_backprop_lolu(_ptr(gatec), _ptr(wn), _ptr(drg), _ptr(want_gate), _ptr(dwn), len_moe, X)
    orc.lib.orc_normalize_state_backward(_ptr(widec), _ptr(dwn), _ptr(want_vals), len_moe, X, tiles)
    live = host["sid"] >= 0
    got_gate = d_gate.float().cpu().numpy(); got_vals = d_vals.float().cpu().numpy(); got_w = dxw.cpu().numpy()
    # padding rows (routing weight 0) give zeros
    assert (got_gate[~live] == 0).all() and (got_vals[~live] == 0).all() and (got_w[~live] == 0).all()
    # bf16 results: half an ulp (2^-9 relative) plus the fp32 noise of the chain
    for got, want, what in ((got_gate, want_gate, "dgate"), (got_vals, want_vals, "dwide")):
        err = np.abs(got[live] - want[live])
        assert (err <= 4.2e-3 * np.abs(want[live]) + 2e-5 * np.abs(want[live]).max()).all(), (what, err.max())
    np.testing.assert_allclose(got_w[live], grad_moe[live, 0], rtol=2e-5, atol=2e-5 * np.abs(grad_moe).max())
    assert (got_vals[5, 128:256] == 0).all()


def offset_view(t, elems=4):
    """the same values at a base address that is 8 bytes off a 16-byte boundary: the entry points then take their four-element kernels"""
    rows, cols = t.shape
    buf = torch.zeros((rows, cols + 2 * elems), dtype=t.dtype, device=t.device)
    view = buf[:, elems:elems + cols]
    view.copy_(t)
    assert view.data_ptr() % 16 == 8 and (view.stride(0) * view.element_size()) % 16 == 0
    return view


def e4m3_steps(orc, a, b):
    """distance of two arrays of e4m3 codes in grid steps (positions on the sorted grid of the 254 finite values)"""
    tab = orc.e4m3_table(hw=True).astype(np.float64)
    fin = np.isfinite(tab)
    order = np.full(256, -1, np.int64)
    vals = np.unique(tab[fin])
    order[fin] = np.searchsorted(vals, tab[fin])
    assert (order[a] >= 0).all() and (order[b] >= 0).all()
    return np.abs(order[a] - order[b])


@pytest.mark.parametrize("X", [256, 1024])
def test_lolu_moe_e4m3_sixteen_wide_kernel_equals_the_four_wide_kernel(lib, X):
    """ts2_matrix_lolu_moe with an e4m3 result and 16-byte aligned operands runs the kernel of sixteen elements per lane; the same values
    at an address 8 bytes off run the four-element kernel, itself checked against MatrixLoLUmoe of the CPU layer by the model tests.
    Same arithmetic per element: the codes are equal."""
    L = lib
    len_, E, K = 700, 64, 2
    print("case moe lolu e4m3", X, flush=True)
    _, t, tb, len_moe, host = route(L, len_, E, K, 31)
    r = np.random.default_rng(32)
    gate = torch.from_numpy((r.standard_normal((len_moe, X)) * 1.5).astype(np.float32)).cuda().bfloat16()
    vals = torch.from_numpy((r.standard_normal((len_moe, X)) * 24).astype(np.float32)).cuda().bfloat16()
    fast = torch.full((len_moe, X), 0x55, dtype=torch.uint8, device="cuda")
    slow = torch.full((len_moe, X), 0x55, dtype=torch.uint8, device="cuda")
    L.call("ts2_matrix_lolu_moe", len_moe, t["sw"], gate, vals, 0.75, fast, L.E4M3)
    L.call("ts2_matrix_lolu_moe", len_moe, t["sw"], offset_view(gate), offset_view(vals), 0.75, slow, L.E4M3)
    torch.cuda.synchronize()
    f, s = fast.cpu().numpy(), slow.cpu().numpy()
    live = host["sid"] >= 0
    assert np.array_equal(f, s)
    assert (f[~live] == 0).all() and (f[live] != 0).mean() > 0.9
    # and the values: vals * sigmoid(2 gate) * weight * 0.75, rounded to e4m3 (half a step of three mantissa bits)
    orc = Oracle()
    got = orc.e4m3_table(hw=True)[f[live]]
    g = gate.float().cpu().numpy()[live]; v = vals.float().cpu().numpy()[live]
    want = np.clip(v / (1 + np.exp(-2 * g.astype(np.float64))) * host["sw"][live][:, None] * 0.75, -448, 448)  # the conversion saturates
    assert (np.abs(got - want) <= np.abs(want) * 2.0 ** -4 + 2.0 ** -10).all()


@pytest.mark.parametrize("X", [256, 1024])
def test_gate_and_norm_backward_e4m3_wave_kernel_equals_the_generic_kernel(lib, X):
    """bf16 gradient in, e4m3 out (the fp8 model's types) runs the wave-per-row kernel; X = 1024 takes its tile loop twice, X = 256 leaves
    half of each wave without a tile.  The same values at an address 8 bytes off run the generic kernel (checked against the CPU layer
    above).  Per element the same arithmetic; the two 128-element tile sums are formed in a different order, so a code may move by one
    step where a value sits on a rounding boundary, and the routing-weight gradient agrees to fp32 summation noise."""
    L = lib
    orc = Oracle()
    len_, E, K = 700, 64, 2
    print("case moe gate/norm backward e4m3", X, flush=True)
    _, t, tb, len_moe, host = route(L, len_, E, K, 33)
    r = np.random.default_rng(34)
    tiles = X // 128
    vals16 = torch.from_numpy((r.standard_normal((len_moe, X)) * 24).astype(np.float32)).cuda().bfloat16()
    vals16[7, 128:256] = 0  # a zero tile
    gate16 = torch.from_numpy((r.standard_normal((len_moe, X)) * 1.5).astype(np.float32)).cuda().bfloat16()
    grad = torch.from_numpy((r.standard_normal((len_moe, X)) * 16).astype(np.float32)).cuda().bfloat16()
    tsc = torch.from_numpy(np.exp(r.standard_normal((tiles, len_moe))).astype(np.float32)).cuda()
    outs = []
    for off in (False, True):
        d_gate = torch.full((len_moe, X), 0x55, dtype=torch.uint8, device="cuda"); d_vals = torch.full_like(d_gate, 0x55)
        dxw = torch.full((len_moe,), 9.0, device="cuda")
        g, v, gr = (offset_view(x) if off else x for x in (gate16, vals16, grad))
        L.call("ts2_backprop_row_tile_normalize_lolu_moe", len_moe, t["sw"], g, v, float(VEC), tsc, gr, L.BF16, 0.5, d_gate, d_vals, L.E4M3, dxw)
        torch.cuda.synchronize()
        outs.append((d_gate.cpu().numpy(), d_vals.cpu().numpy(), dxw.cpu().numpy()))
    (fg, fv, fw), (sg, sv, sw) = outs
    live = host["sid"] >= 0
    assert (fg[~live] == 0).all() and (fv[~live] == 0).all() and (fw[~live] == 0).all()
    assert np.array_equal(fg, sg)                      # no reduction enters the gate gradient
    steps = e4m3_steps(orc, fv, sv)
    assert steps.max() <= 1 and (steps != 0).mean() < 2e-3, (steps.max(), (steps != 0).mean())
    assert (fv[7, 128:256] == 0).all() and (fv[live] != 0).mean() > 0.9
    np.testing.assert_allclose(fw, sw, rtol=2e-5, atol=2e-5 * np.abs(sw).max())


@pytest.mark.parametrize("selected", [1, 3, 4, 5, 6])
def test_combine_experts_bf16_slot_counts(lib, selected):
    """bf16 grouped rows: up to four selected experts take the kernel with four tokens per lane (902 tokens: its last group of four is
    half empty), more than four the kernel that gathers the slots in batches of four and takes a second batch.
    The sum is in slot order, as numpy's."""
    L = lib
    len_, E, dim = 902 if selected < 5 else 900, 16, 512  # 902: the last group of four tokens is half empty
    print("case moe combine bf16 slots", selected, flush=True)
    _, t, tb, len_moe, host = route(L, len_, E, selected, 35)
    r = np.random.default_rng(36)
    src = torch.from_numpy(r.standard_normal((len_moe, dim)).astype(np.float32)).cuda().bfloat16()
    srcf = src.float().cpu().numpy()
    res0 = r.standard_normal((len_, dim)).astype(np.float32)
    alpha = np.float32(0.37)
    ap = torch.tensor([1.5], device="cuda")
    s = alpha * np.float32(1.5)
    for add in (0, 1):
        res = torch.from_numpy(res0.copy()).cuda()
        L.call("ts2_combine_experts", len_, selected, src, L.BF16, C.byref(tb), float(alpha), ap, res, add)
        res4 = torch.from_numpy(res0.copy()).cuda()
        L.call("ts2_combine_experts", len_, selected, offset_view(src), L.BF16, C.byref(tb), float(alpha), ap, res4, add)
        torch.cuda.synchronize()
        want = np.zeros((len_, dim), np.float32)
        for k in range(selected):
            want = want + srcf[host["row"][:, k]]
        want = want * s
        if add:
            want = want + res0
        assert np.array_equal(res.cpu().numpy(), want), add
        assert np.array_equal(res4.cpu().numpy(), want), add
