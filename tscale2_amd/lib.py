"""ctypes view of include/ts2_abi.h.  Device memory and streams come from torch (plumbing only); every compute call goes
through the C ABI of libts2amd.so.  There is no fallback: a missing library is an error."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
SO = os.path.join(HERE, "libts2amd.so")

I8, E4M3, BF16, F32, I32 = 0, 1, 2, 3, 4
EPI_STORE, EPI_ADD, EPI_ROW_TILE_MAXNORM = 0, 1, 2


class Mat(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("strideBytes", C.c_int64), ("x", C.c_int32), ("y", C.c_int32)]


class GemmArgs(C.Structure):
    _fields_ = [("a", Mat), ("b", Mat), ("c", Mat), ("abType", C.c_int32), ("cType", C.c_int32), ("m", C.c_int32), ("n", C.c_int32),
                ("k", C.c_int32), ("mLive", C.c_int32), ("rowScale", C.c_void_p), ("kTileScale", C.c_void_p), ("kTile", C.c_int32),
                ("alpha", C.c_float), ("alphaPtr", C.c_void_p), ("epilogue", C.c_int32), ("tileScale", Mat), ("splitK", C.c_int32),
                ("tileConfig", C.c_int32)]


def mat(t):
    """2-D view of a torch tensor (row-major, last dim contiguous)."""
    if t is None:
        return Mat(None, 0, 0, 0)
    assert t.dim() == 2 and t.stride(1) == 1, "ts2_mat needs a row-major 2-D tensor"
    return Mat(t.data_ptr(), t.stride(0) * t.element_size(), t.shape[1], t.shape[0])


def ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


class Lib:
    def __init__(self, path=SO):
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it with `python -m tscale2_amd.build` (no CPU fallback exists)")
        self.dll = C.CDLL(path)
        self.dll.ts2_version.restype = C.c_char_p

    def __getattr__(self, name):
        return getattr(self.dll, name)

    @staticmethod
    def stream():
        import torch
        return C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def check(self, rc, what):
        if rc != 0:
            raise RuntimeError(f"{what} failed with code {rc}")

    def gemm_nt(self, a, b, c, ab_type, c_type, row_scale=None, k_tile_scale=None, k_tile=0, alpha=1.0, alpha_ptr=None,
                epilogue=EPI_STORE, tile_scale=None, split_k=1, m_live=0, tile_config=0, k=None, check=True):
        args = GemmArgs()
        args.a, args.b, args.c = mat(a), mat(b), mat(c)
        args.abType, args.cType = ab_type, c_type
        args.m, args.n = a.shape[0], b.shape[0]
        args.k = a.shape[1] if k is None else k
        args.mLive = m_live
        args.rowScale = ptr(row_scale)
        args.kTileScale = ptr(k_tile_scale)
        args.kTile = k_tile
        args.alpha = alpha
        args.alphaPtr = ptr(alpha_ptr)
        args.epilogue = epilogue
        args.tileScale = mat(tile_scale)
        args.splitK = split_k
        args.tileConfig = tile_config
        rc = self.dll.ts2_gemm_nt(C.byref(args), self.stream())
        if check:
            self.check(rc, "ts2_gemm_nt")
        return rc


_lib = None


def load():
    global _lib
    if _lib is None:
        _lib = Lib()
    return _lib


def _conv(a, keep):
    """torch 2-D tensor -> ts2_mat*, 1-D/0-D tensor -> raw device pointer, float -> c_float, int -> c_int32, None -> NULL."""
    import torch
    if a is None:
        return None
    if isinstance(a, torch.Tensor):
        if a.dim() == 2:
            m = mat(a)
            keep.append(m)
            return C.byref(m)
        return C.c_void_p(a.data_ptr())
    if isinstance(a, bool):
        return C.c_int32(int(a))
    if isinstance(a, int):
        return C.c_int32(a)
    if isinstance(a, float):
        return C.c_float(a)
    return a


def call(name, *args, check=True):
    """Invoke an entry point of the C ABI on torch's current stream (appended as the last argument)."""
    lib = load()
    keep = []
    cargs = [_conv(a, keep) for a in args]
    rc = getattr(lib.dll, name)(*cargs, lib.stream())
    if check and rc != 0:
        raise RuntimeError(f"{name} failed with code {rc}")
    return rc
