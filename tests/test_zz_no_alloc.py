"""ts2_moe_route_static (the routing entry point that allocates nothing and keeps its scratch in a fixed device array) against
ts2_moe_route with a caller-owned workspace: every table bit-identical, on two calls in a row, the second with a smaller input."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

NAMES = ("ids", "w", "off", "eo", "tile", "sid", "sw", "bc")


class Tables(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in NAMES]


def make_tables(len_, experts, selected, with_workspace):
    total = len_ * selected
    len_moe = (total + 128 * experts + 127) // 128 * 128
    dev = "cuda"
    # filled with a pattern so that stale contents cannot pass for results
    t = {"ids": torch.full((total,), -7, dtype=torch.int32, device=dev), "w": torch.full((total,), -7.0, device=dev),
         "off": torch.full((total,), -7, dtype=torch.int32, device=dev), "eo": torch.full((experts + 2,), -7, dtype=torch.int32, device=dev),
         "tile": torch.full((len_moe // 128,), -7, dtype=torch.int32, device=dev), "sid": torch.full((len_moe,), -7, dtype=torch.int32, device=dev),
         "sw": torch.full((len_moe,), -7.0, device=dev)}
    if with_workspace:
        t["bc"] = torch.full((((total + 255) // 256) * experts,), -7, dtype=torch.int32, device=dev)
    tb = Tables(*[t[n].data_ptr() if n in t else None for n in NAMES])
    return t, tb, len_moe


def route_both(L, len_, experts, selected, seed):
    r = np.random.default_rng(seed)
    sel = torch.from_numpy(r.standard_normal((len_, experts)).astype(np.float32)).cuda()
    ta, tba, len_moe = make_tables(len_, experts, selected, True)
    tb_, tbb, _ = make_tables(len_, experts, selected, False)
    L.call("ts2_moe_route", len_, len_moe, experts, selected, sel, L.F32, C.byref(tba))
    L.call("ts2_moe_route_static", len_, len_moe, experts, selected, sel, L.F32, C.byref(tbb))
    torch.cuda.synchronize()
    for n in NAMES[:-1]:
        a, b = ta[n].cpu().numpy(), tb_[n].cpu().numpy()
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), (n, len_, experts, selected)
    # the tables are real results, not the fill pattern
    eo = ta["eo"].cpu().numpy()
    assert eo[0] == 0 and eo[experts + 1] == len_moe and (ta["sid"].cpu().numpy() >= 0).sum() == len_ * selected


def test_static_scratch_routing_equals_workspace_routing_on_consecutive_calls():
    from tscale2_amd import lib as L
    L.load()
    print("case moe route static: 40000 x 64 top-2, then 3000 x 8 top-2, then 517 x 64 top-3", flush=True)
    route_both(L, 40000, 64, 2, 11)  # 313 counting blocks x 64 experts of scratch
    route_both(L, 3000, 8, 2, 12)    # smaller: the array still holds the first call's counts
    route_both(L, 517, 64, 3, 13)


def test_static_scratch_routing_rejects_sizes_beyond_its_array():
    from tscale2_amd import lib as L
    L.load()
    len_, experts, selected = 140000, 256, 2  # 1094 blocks x 256 experts = 280064 ints > 131072
    sel = torch.zeros((len_, experts), device="cuda")
    t, tb, len_moe = make_tables(len_, experts, selected, False)
    rc = L.call("ts2_moe_route_static", len_, len_moe, experts, selected, sel, L.F32, C.byref(tb), check=False)
    assert rc == -1  # TS2_ERR_SHAPE
    torch.cuda.synchronize()
    assert int(t["eo"][0].item()) == -7  # nothing ran
