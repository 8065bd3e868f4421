"""MI355X (gfx950) backward path for the TScale2 transformer trainer: hand-written HIP kernels behind a C ABI.
This Python package is only the loader used by tests and benchmarks; the product is tscale2_amd/libts2amd.so."""
from .lib import Lib, load  # noqa: F401
