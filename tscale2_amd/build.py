"""Builds tscale2_amd/libts2amd.so (all HIP kernels + the C ABI) and tscale2_amd/libts2probe.so (the benchmark's machine probes) for
gfx950 with hipcc.  No GPU is needed to build."""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libts2amd.so")
PROBE_OUT = os.path.join(HERE, "libts2probe.so")
OBJ = os.path.join(HERE, "build")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-I", os.path.join(os.path.dirname(HERE), "include")]


def _compile(src):
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    r = subprocess.run(["hipcc", *FLAGS, "-c", src, "-o", obj], capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.cpp")))
    probes = sorted(glob.glob(os.path.join(CSRC, "probe", "*.hip")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, srcs + probes))
    for out, o in ((OUT, objs[:len(srcs)]), (PROBE_OUT, objs[len(srcs):])):
        r = subprocess.run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out, *o], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stderr)
    return OUT


if __name__ == "__main__":
    print(build())
