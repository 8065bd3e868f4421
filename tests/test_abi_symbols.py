"""The C-ABI libraries load without a GPU and export every entry point that include/*.h declares (no compute call is made)."""
import ctypes as C
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ts2_abi.h")
SO = os.path.join(ROOT, "tscale2_amd", "libts2amd.so")
PROBE_HEADER = os.path.join(ROOT, "include", "ts2_probe.h")
PROBE_SO = os.path.join(ROOT, "tscale2_amd", "libts2probe.so")


def declared_functions(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    return sorted(set(re.findall(r"\b(ts2_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_hot_path():
    names = declared_functions()
    for must in ("ts2_gemm_nt", "ts2_matmul_backprop_multi", "ts2_matmul_backprop", "ts2_matmul_backprop_delta", "ts2_att_backward",
                 "ts2_backprop_layer_normalize", "ts2_scale_grad", "ts2_backprop_moe", "ts2_combine_experts", "ts2_model_backprop"):
        assert must in names


def test_library_exports_every_declared_symbol():
    assert os.path.exists(SO), "build the library first: python -m tscale2_amd.build"
    dll = C.CDLL(SO)
    missing = [n for n in declared_functions() if not hasattr(dll, n)]
    assert not missing, missing
    dll.ts2_version.restype = C.c_char_p
    assert dll.ts2_version().decode().startswith("ts2amd")


def test_probe_library_exports_its_header_and_the_product_header_holds_no_probe():
    assert not [n for n in declared_functions() if "probe" in n]
    assert os.path.exists(PROBE_SO), "build the library first: python -m tscale2_amd.build"
    dll = C.CDLL(PROBE_SO)
    names = declared_functions(PROBE_HEADER)
    assert names == ["ts2_probe_clock_monitor", "ts2_probe_copy_rate", "ts2_probe_mfma_rate"]
    assert not [n for n in names if not hasattr(dll, n)]


def test_scratch_size_query_of_the_linear_backward_operator():
    dll = C.CDLL(SO)
    out = (C.c_int64 * 9)()
    assert dll.ts2_matmul_bwd_scratch_bytes(0, 16384, 1024, 4096, 512, 2, out) == 0  # int8, config[1]
    assert list(out) == [16384 * 4096, 16384 * 4, 4096 * 16384, 1024 * 16384, 32 * 4, 32 * 4, 1024 * 4096, 2 * 4096 * 1024 * 4, 16384 * 4]
    assert dll.ts2_matmul_bwd_scratch_bytes(1, 32768, 2048, 8192, 0, 1, out) == 0  # e4m3: no row-quantised copy, no k-tile scales
    assert list(out) == [0, 0, 8192 * 32768, 2048 * 32768, 0, 0, 2048 * 8192, 0, 0]
    assert dll.ts2_matmul_bwd_scratch_bytes(0, 16384, 1000, 4096, 512, 1, out) == -1
    assert dll.ts2_matmul_bwd_scratch_bytes(2, 16384, 1024, 4096, 512, 1, out) == -3


def test_batch_validation_rejects_out_of_range_indices():
    """every index the device kernels follow (labels, targets, spans) is refused on the host when it is out of range"""
    import numpy as np
    dll = C.CDLL(SO)
    n, label_count, vocab = 6, 10, 8

    def run(label_ptr=None, labels=None, target=None, start=None, finish=None, label_cap=64):
        lp = np.arange(n + 1, dtype=np.int32) if label_ptr is None else np.asarray(label_ptr, np.int32)
        lb = np.arange(1, n + 1, dtype=np.uint32) if labels is None else np.asarray(labels, np.uint32)
        tg = np.array([1, 2, 3, 4, 5, -1], np.int32) if target is None else np.asarray(target, np.int32)
        st = np.zeros(n, np.int32) if start is None else np.asarray(start, np.int32)
        fi = np.arange(-1, n - 1, dtype=np.int32) if finish is None else np.asarray(finish, np.int32)
        ps = (C.c_void_p * 1)(st.ctypes.data)
        pf = (C.c_void_p * 1)(fi.ctypes.data)
        return dll.ts2_validate_batch(n, label_cap, label_count, vocab, 1, lp.ctypes.data_as(C.c_void_p), lb.ctypes.data_as(C.c_void_p),
                                      tg.ctypes.data_as(C.c_void_p), ps, pf)

    assert run() == 0
    assert run(labels=[1, 2, 3, 4, 5, 0x80000000 | 9]) == 0      # negative-sign label with a valid id
    assert run(labels=[1, 2, 3, 4, 5, 10]) == -1                 # label id == labelCount
    assert run(labels=[1, 2, 3, 4, 5, 0x80000000 | 10]) == -1
    assert run(target=[1, 2, 3, 4, 8, -1]) == -1                 # target == vocab
    assert run(target=[1, 2, 3, 4, -2, -1]) == -1
    assert run(label_ptr=[0, 1, 2, 2, 1, 5, 6]) == -1            # CSR not monotone
    assert run(label_ptr=[1, 1, 2, 3, 4, 5, 6]) == -1            # CSR does not start at 0
    assert run(label_cap=5) == -1                                # more labels than the model holds
    assert run(start=[0, 0, 0, 0, 0, -1]) == -1                  # span starts before row 0
    assert run(finish=[-1, 0, 1, 2, 3, 6]) == -1                 # span ends beyond the batch
    assert run(start=[0, 0, 0, 0, 0, 5], finish=[-1, 0, 1, 2, 3, 2]) == 0   # finish < start: an empty span
    assert run(finish=[-2, 0, 1, 2, 3, 4]) == -1                 # finish below -1
    assert run(start=[0, 0, 0, 0, 0, 7]) == -1                   # start beyond the batch


def test_every_entry_point_cites_the_interface_it_replaces():
    """each declaration is preceded by a comment naming a reference file:line, or says that it has no counterpart there"""
    text = open(HEADER).read()
    assert len(re.findall(r"[a-z_]+\.(?:cuh|cu|h|cpp):\d+", text)) >= 30


def test_model_schedule_and_rope_table_equal_the_oracle():
    """ts2_model_schedule / ts2_fill_rope_buf (host code of the library) against the oracle's restatements, which are bit-exact against
    the reference build (tests/test_oracle_vs_reference.py): InitAlibi src/gpt/model_params/model_dim.cpp:82-158, FillRopeBuf
    src/gpt/att/rope.cpp:4-38.  No GPU needed."""
    import numpy as np
    from oracle_lib import Oracle
    from tscale2_amd import lib as L
    orc = Oracle()
    for depth, experts, wide in ((1, 0, 64), (1, 8, 256), (2, 0, 64), (3, 8, 64), (12, 0, 1024), (13, 0, 128), (24, 16, 512), (60, 0, 64)):
        want = orc.model_schedule(None, depth, experts, wide)
        lt, la, ls, aw = L.model_schedule(depth, experts, wide)
        assert np.array_equal(lt, want["layer_type"]) and np.array_equal(la, want["layer_att_id"]), (depth, experts)
        assert np.array_equal(ls, want["layer_slope"]) and np.array_equal(aw, want["att_width"]), (depth, experts)
    for width, n in ((128, 300), (64, 17), (128, 2048)):
        assert np.array_equal(L.fill_rope_buf(width, n), orc.fill_rope_buf(width, n))
