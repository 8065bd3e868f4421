"""The C-ABI library loads without a GPU and exports every entry point that include/ts2_abi.h declares (no compute call is made)."""
import ctypes as C
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ts2_abi.h")
SO = os.path.join(ROOT, "tscale2_amd", "libts2amd.so")


def declared_functions():
    text = open(HEADER).read()
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


def test_every_entry_point_cites_the_interface_it_replaces():
    """each declaration is preceded by a comment naming a reference file:line, or says that it has no counterpart there"""
    text = open(HEADER).read()
    assert len(re.findall(r"[a-z_]+\.(?:cuh|cu|h|cpp):\d+", text)) >= 30
