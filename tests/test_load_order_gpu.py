"""The ctypes view must work whichever of torch and the library a program imports first."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

PROGRAM = """
import sys
sys.path.insert(0, %r)
from tscale2_amd import lib as L
L.load()                       # before this program has imported torch
import torch
x = torch.randn((256, 256), device="cuda")
out = torch.empty((256, 256), dtype=torch.uint8, device="cuda")
scale = torch.empty((2, 256), device="cuda")
L.call("ts2_layer_normalize_state_vecs", x, L.F32, 256, 256, 1 / 24, out, L.E4M3, scale)
torch.cuda.synchronize()
v = out.view(torch.float8_e4m3fn).float()
assert abs(float((v * v).mean()) - 576.0) < 30.0, float((v * v).mean())
print("launch ok")
"""


@pytest.mark.gpu
def test_library_loaded_before_torch_still_launches():
    """a process that loads the library before it imports torch: the wrapper pulls torch (and with it torch's HIP runtime) in first, so
    the kernels are registered with the runtime that owns the tensors"""
    print("case load order", flush=True)
    r = subprocess.run([sys.executable, "-c", PROGRAM % ROOT], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "launch ok" in r.stdout, r.stdout[-500:] + r.stderr[-1500:]
