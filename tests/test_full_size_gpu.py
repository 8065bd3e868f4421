"""The kernels at the full sizes of the benchmark configurations, checked through properties that need no CPU reference of that size:
row/column checksums of a product (exact for int32-accumulated int8), independence of the sequences of a causal batch, and
linearity of dK/dV in dO."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def L():
    from tscale2_amd import lib
    lib.load()
    return lib


def checksums(a, b):
    """sum_i C[i][j] and sum_j C[i][j] of C = A B^T from the operand sums, in float64 (exact below 2^53)"""
    a64, b64 = a.double(), b.double()
    col = (a64.sum(0, keepdim=True) @ b64.t()).ravel()      # [n]
    row = (a64 @ b64.sum(0, keepdim=True).t()).ravel()      # [m]
    return col, row


@pytest.mark.parametrize("m,n,k", [(16384, 1024, 4096), (4096, 1024, 16384)])
def test_int8_products_of_the_linear_backward_are_exact_at_full_size(L, m, n, k):
    """config[1]: dX is [16384 x 4096] x [1024 x 4096]^T, the delta [4096 x 16384] x [1024 x 16384]^T; every row sum and every column sum
    of the int32 result must equal the value computed from the operand sums -- bit-exact"""
    print("case int8 full size", m, n, k, flush=True)
    lib = L.load()
    g = torch.Generator(device="cuda").manual_seed(m + k)
    a = torch.randint(-127, 128, (m, k), dtype=torch.int8, device="cuda", generator=g)
    b = torch.randint(-127, 128, (n, k), dtype=torch.int8, device="cuda", generator=g)
    c = torch.empty((m, n), dtype=torch.int32, device="cuda")
    lib.gemm_nt(a, b, c, L.I8, L.I32)
    col, row = checksums(a, b)
    c64 = c.double()
    assert torch.equal(c64.sum(0), col)
    assert torch.equal(c64.sum(1), row)
    # one row recomputed directly
    i = 12345 % m
    assert torch.equal(c[i].double(), b.double() @ a[i].double())


def test_fp8_product_at_the_size_of_the_dense_model(L):
    """config[2]: the FFN dX product 32768 x 2048 x 8192 in e4m3 with fp32 accumulation; checksums within 1e-4 of the largest one"""
    print("case fp8 full size", flush=True)
    lib = L.load()
    m, n, k = 32768, 2048, 8192
    g = torch.Generator(device="cuda").manual_seed(3)
    a = (torch.randn((m, k), device="cuda", generator=g) * 4).to(torch.float8_e4m3fn)
    b = (torch.randn((n, k), device="cuda", generator=g) * 4).to(torch.float8_e4m3fn)
    c = torch.empty((m, n), dtype=torch.float32, device="cuda")
    lib.gemm_nt(a.view(torch.uint8), b.view(torch.uint8), c, L.E4M3, L.F32)
    col, row = checksums(a.float(), b.float())
    c64 = c.double()
    # a checksum adds m (or n) results whose rounding errors (about 4e-5 of the row's largest partial sum each) are independent
    scale = c64.abs().max().item()
    assert (c64.sum(0) - col).abs().max().item() <= 1e-4 * scale * np.sqrt(m)
    assert (c64.sum(1) - row).abs().max().item() <= 1e-4 * scale * np.sqrt(n)
    i = 777
    ref = b.double() @ a[i].double()
    assert (c[i].double() - ref).abs().max().item() <= 2e-4 * ref.abs().max().item()


def test_fp8_delta_product_on_untransposed_operands_at_the_size_of_the_dense_model(L):
    """config[2]: the delta of the FFN expand matrix, 8192 x 2048 over 32768 tokens, contracting over the rows of the gradient
    [token][8192] and the layer input [token][2048] as they lie (kMajor).  fp32 store: checksums within 1e-4 of the largest result
    times sqrt(count), one row recomputed directly; the packed delta (what the operator stores) dequantised within 1/254 of each
    row tile's maximum of the fp32 result."""
    print("case fp8 K-major delta full size", flush=True)
    lib = L.load()
    m, n, k = 8192, 2048, 32768
    g = torch.Generator(device="cuda").manual_seed(4)
    a = (torch.randn((k, m), device="cuda", generator=g) * 2).to(torch.float8_e4m3fn)     # gradient [token][m]
    b = (torch.randn((k, n), device="cuda", generator=g) * 2).to(torch.float8_e4m3fn)     # input [token][n]
    c = torch.empty((m, n), dtype=torch.float32, device="cuda")
    lib.gemm_nt(a.view(torch.uint8), b.view(torch.uint8), c, L.E4M3, L.F32, m=m, n=n, k=k, k_major=True)
    a64sum, b64sum = a.double().sum(1), b.double().sum(1)                                   # per token
    col = (a64sum.unsqueeze(0) @ b.double()).ravel()                                        # sum_i C[i][j]
    row = (a.double().t() @ b64sum.unsqueeze(1)).ravel()                                    # sum_j C[i][j]
    c64 = c.double()
    scale = c64.abs().max().item()
    assert (c64.sum(0) - col).abs().max().item() <= 1e-4 * scale * np.sqrt(m)
    assert (c64.sum(1) - row).abs().max().item() <= 1e-4 * scale * np.sqrt(n)
    i = 4321
    ref = a[:, i].double() @ b.double()
    assert (c[i].double() - ref).abs().max().item() <= 2e-4 * ref.abs().max().item()
    d8 = torch.empty((m, n), dtype=torch.int8, device="cuda")
    ts = torch.empty((n // 128, m), device="cuda")
    lib.gemm_nt(a.view(torch.uint8), b.view(torch.uint8), d8, L.E4M3, L.I8, epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=ts, m=m, n=n, k=k,
                k_major=True)
    torch.cuda.synchronize()
    deq = d8.float().view(m, n // 128, 128) * ts.t().unsqueeze(2)
    tile_max = c.view(m, n // 128, 128).abs().amax(2, keepdim=True)
    assert ((deq - c.view(m, n // 128, 128)).abs() <= tile_max / 254 * 1.0001 + 1e-30).all()
    assert torch.allclose(ts.t(), tile_max.squeeze(2) / 127, rtol=1e-6)


def test_attention_at_full_size_treats_the_sequences_of_a_batch_independently(L):
    """config[3]: 16 sequences x 2048 tokens, 16 heads.  Forward, dQ, dK and dV of one sequence taken from the batch run equal, bit
    for bit, the run of that sequence alone (same tiles, same order of operations); dK/dV are linear in dO."""
    print("case attention full size", flush=True)
    B, S, H = 16, 2048, 16
    n = B * S
    i16 = torch.int16
    g = torch.Generator(device="cuda").manual_seed(9)
    q, k, v, do = [torch.randn((n, H * 128), device="cuda", generator=g).bfloat16() for _ in range(4)]
    sc = 0.0637

    def run(q, k, v, do, n, slope):
        t = torch.arange(n, device="cuda", dtype=torch.int32)
        start = ((t // S) * S).int().contiguous()
        finish = torch.where(t - 1 >= start, t - 1, torch.full_like(t, -1)).int().contiguous()
        val = torch.empty_like(q)
        swl = torch.empty((H, n), device="cuda")
        rl = torch.zeros(n // 128, dtype=torch.int32, device="cuda")
        rh = torch.zeros_like(rl)
        L.call("ts2_att_build_rev", n, n, start, finish, rl, rh)
        L.att_forward(n, H, q.view(i16), k.view(i16), v.view(i16), start, finish, sc, slope, val.view(i16), swl)
        ds = (val.float() * do.float()).view(n, H, 128).sum(-1).t().contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
        L.att_backward(n, H, q.view(i16), k.view(i16), v.view(i16), do.view(i16), start, finish, rl, rh, sc, slope, swl, ds, dq.view(i16), dk.view(i16),
                       dv.view(i16), L.BF16, 3)
        return val, swl, dq, dk, dv, ds, (start, finish, rl, rh)

    slope = 0.01
    val, swl, dq, dk, dv, ds, aux = run(q, k, v, do, n, slope)
    for t in (val, dq, dk, dv):
        assert torch.isfinite(t.float()).all()
    s = 5
    sl = slice(s * S, (s + 1) * S)
    val1, swl1, dq1, dk1, dv1, _, _ = run(q[sl].contiguous(), k[sl].contiguous(), v[sl].contiguous(), do[sl].contiguous(), S, slope)
    assert torch.equal(val[sl].view(i16), val1.view(i16))
    assert torch.equal(swl[:, sl], swl1)
    assert torch.equal(dq[sl].view(i16), dq1.view(i16))
    assert torch.equal(dk[sl].view(i16), dk1.view(i16))
    assert torch.equal(dv[sl].view(i16), dv1.view(i16))
    # the first token of a sequence sees nothing: output 0, statistics of the sink alone, no gradient to its query
    assert (val[s * S].float() == 0).all() and (swl[:, s * S] == 0).all() and (dq[s * S].float() == 0).all()
    # the last key of a sequence is seen by no query: no gradient
    assert (dk[(s + 1) * S - 1].float() == 0).all() and (dv[(s + 1) * S - 1].float() == 0).all()
    # dV is linear in dO (for fixed probabilities): dV(2 dO) = 2 dV(dO) exactly in bf16, since scaling by two is exact
    start, finish, rl, rh = aux
    do2 = (do.float() * 2).bfloat16()
    dq2, dk2, dv2 = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    L.att_backward(n, H, q.view(i16), k.view(i16), v.view(i16), do2.view(i16), start, finish, rl, rh, sc, slope, swl, (ds * 2).contiguous(), dq2.view(i16),
                   dk2.view(i16), dv2.view(i16), L.BF16, 3)
    assert torch.equal(dv2.float(), dv.float() * 2)
    assert torch.equal(dk2.float(), dk.float() * 2)
    assert torch.equal(dq2.float(), dq.float() * 2)


def test_moe_routing_gather_grouped_product_and_combine_at_the_size_of_the_moe_benchmark(L):
    """config[4]: 65536 tokens routed to 2 of 64 experts (139264 grouped rows with every expert's rows padded to 128), width 1024, expert
    width 512.  Routing tables by their invariants, ts2_moe_group_samples against a torch gather (bit-exact), the expert-grouped e4m3
    product 139264 x 512 x 1024 through per-expert row and column checksums in float64, ts2_combine_experts against a torch gather-sum
    (bit-exact).  Reference: src/gpt/compute/layer_moe.cu:203-272 (forward), moe_matmul.cuh:47-215 (grouped products)."""
    import ctypes as C
    from test_moe_gpu import route
    print("case moe full size", flush=True)
    lib = L.load()
    len_, E, K, dim, xp = 65536, 64, 2, 1024, 512
    _, t, tb, len_moe, host = route(L, len_, E, K, 61)
    assert len_moe == 139264
    sid, eo, tile = t["sid"].long(), host["eo"], host["tile"]
    # every token is listed `selected` times, an expert's rows are a multiple of 128, a tile's expert is the owner of its rows
    live = sid >= 0
    assert int(live.sum()) == len_ * K
    assert torch.equal(torch.bincount(sid[live], minlength=len_), torch.full((len_,), K, device="cuda"))
    assert eo[0] == 0 and np.all(np.diff(eo[:E + 1]) % 128 == 0) and np.all(np.diff(eo[:E + 1]) >= 0)
    owner = np.searchsorted(eo[1:E + 1], np.arange(len_moe // 128) * 128, side="right")
    used = np.arange(len_moe // 128) * 128 < eo[E]
    assert np.array_equal(tile[used], owner[used]) and np.all(tile[~used] == -1)
    rows_e = torch.from_numpy(np.repeat(np.where(used, owner, E), 128)).cuda()          # expert of every grouped row (E = unused tail)
    # pad rows (sid -1) lie at the end of each expert's range
    for e in (0, 17, E - 1):
        s = sid[eo[e]:eo[e + 1]]
        nlive = int((s >= 0).sum())
        assert bool((s[:nlive] >= 0).all()) and bool((s[nlive:] < 0).all())
    # ---- gather
    g = torch.Generator(device="cuda").manual_seed(62)
    x8 = (torch.randn((len_, dim), device="cuda", generator=g) * 2).to(torch.float8_e4m3fn).view(torch.uint8)
    grouped = torch.full((len_moe, dim), 77, dtype=torch.uint8, device="cuda")
    L.call("ts2_moe_group_samples", len_moe, 1, x8, t["sid"], grouped)
    want = torch.where(live[:, None], x8[sid.clamp(min=0)], torch.zeros((), dtype=torch.uint8, device="cuda"))
    assert torch.equal(grouped, want)
    # ---- grouped product: every 128-row tile multiplies its expert's [xp x dim] slab
    w8 = (torch.randn((E * xp, dim), device="cuda", generator=g) * 2).to(torch.float8_e4m3fn).view(torch.uint8)
    c = torch.full((len_moe, xp), 5.0, dtype=torch.float32, device="cuda")
    lib.gemm_nt(grouped, w8, c, L.E4M3, L.F32, n=xp, tile_group=t["tile"], b_slab_bytes=xp * dim)
    torch.cuda.synchronize()
    assert bool((c[eo[E]:] == 5.0).all())                                               # skipped tiles leave C alone
    a64 = grouped.view(torch.float8_e4m3fn).double()
    w64 = w8.view(torch.float8_e4m3fn).double().view(E, xp, dim)
    c64 = c.double()
    scale = c64[:eo[E]].abs().max().item()
    # row sums: sum_j C[i][j] = A[i] . (sum_j W_e[j])
    wsum = torch.cat([w64.sum(1), torch.zeros((1, dim), dtype=torch.float64, device="cuda")])     # [E + 1][dim]
    row = (a64 * wsum[rows_e]).sum(1)
    assert (c64[:eo[E]].sum(1) - row[:eo[E]]).abs().max().item() <= 1e-4 * scale * np.sqrt(xp)
    # column sums per expert: sum_{i in e} C[i][j] = (sum_{i in e} A[i]) . W_e[j]
    asum = torch.zeros((E + 1, dim), dtype=torch.float64, device="cuda").index_add_(0, rows_e, a64)
    csum = torch.zeros((E + 1, xp), dtype=torch.float64, device="cuda").index_add_(0, rows_e[:eo[E]], c64[:eo[E]])
    col = torch.einsum("ed,exd->ex", asum[:E], w64)
    per_expert = np.diff(eo[:E + 1]).max()
    assert (csum[:E] - col).abs().max().item() <= 1e-4 * scale * np.sqrt(per_expert)
    # one row recomputed directly
    i = int(eo[23]) + 5
    assert (c64[i] - w64[23] @ a64[i]).abs().max().item() <= 2e-4 * scale
    # the same product with a 16-bit result: at this size the library runs it on the persistent kernel with the operands exchanged;
    # same accumulators, so the bf16 rows are the fp32 ones rounded
    c16 = torch.full((len_moe, xp), 0x1234, dtype=torch.int16, device="cuda")
    lib.gemm_nt(grouped, w8, c16, L.E4M3, L.BF16, n=xp, tile_group=t["tile"], b_slab_bytes=xp * dim)
    torch.cuda.synchronize()
    assert bool((c16[eo[E]:] == 0x1234).all())
    assert torch.equal(c16[:eo[E]].view(torch.bfloat16), c[:eo[E]].bfloat16())
    # ---- combine: res = alpha * (*alphaPtr) * sum over a token's slots, in slot order
    src = torch.randn((len_moe, dim), device="cuda", generator=g)
    ap = torch.tensor([1.5], device="cuda")
    res = torch.zeros((len_, dim), device="cuda")
    L.call("ts2_combine_experts", len_, K, src, L.F32, C.byref(tb), 0.37, ap, res, 0)
    torch.cuda.synchronize()
    rows = torch.from_numpy(host["row"]).cuda().long()
    want = (src[rows[:, 0]] + src[rows[:, 1]]) * (np.float32(0.37) * np.float32(1.5))
    assert torch.equal(res, want)
