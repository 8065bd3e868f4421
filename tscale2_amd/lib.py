"""ctypes view of include/ts2_abi.h.  Device memory and streams come from torch (plumbing only); every compute call goes
through the C ABI of libts2amd.so.  There is no fallback: a missing library is an error."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
SO = os.path.join(HERE, "libts2amd.so")
PROBE_SO = os.path.join(HERE, "libts2probe.so")  # the benchmark's machine probes (include/ts2_probe.h), not part of the product ABI

I8, E4M3, BF16, F32, I32, F16 = 0, 1, 2, 3, 4, 5
EPI_STORE, EPI_ADD, EPI_ROW_TILE_MAXNORM, EPI_ROW_TILE_NORM = 0, 1, 2, 3


class Mat(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("strideBytes", C.c_int64), ("x", C.c_int32), ("y", C.c_int32)]


class GemmSegment(C.Structure):
    _fields_ = [("a", C.c_void_p), ("b", C.c_void_p), ("alpha", C.c_float), ("alphaPtr", C.c_void_p)]


class GemmArgs(C.Structure):
    _fields_ = [("a", Mat), ("b", Mat), ("c", Mat), ("abType", C.c_int32), ("cType", C.c_int32), ("m", C.c_int32), ("n", C.c_int32),
                ("k", C.c_int32), ("mLive", C.c_int32), ("rowScale", C.c_void_p), ("kTileScale", C.c_void_p), ("kTile", C.c_int32),
                ("alpha", C.c_float), ("alphaPtr", C.c_void_p), ("epilogue", C.c_int32), ("tileScale", Mat), ("splitK", C.c_int32),
                ("tileConfig", C.c_int32), ("tileGroup", C.c_void_p), ("bSlabBytes", C.c_int64), ("groupOffsets", C.c_void_p),
                ("groups", C.c_int32), ("cSlabBytes", C.c_int64), ("tileScaleSlabBytes", C.c_int64), ("splitSlabBytes", C.c_int64), ("normalize", C.c_int32),
                ("vecScale", C.c_float), ("rope", Mat), ("extraSegments", C.c_int32), ("segment", GemmSegment * 3), ("kMajor", C.c_int32)]


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
        # torch ships its own copy of the HIP runtime.  It has to be in the process before this library is mapped: mapped first, the
        # library binds to the system's copy, the process then holds two runtimes, and launches on torch's tensors fail with
        # "invalid device function" (TS2_ERR_LAUNCH).
        import torch  # noqa: F401
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
                epilogue=EPI_STORE, tile_scale=None, split_k=1, m_live=0, tile_config=0, k=None, check=True, m=None, n=None,
                tile_group=None, b_slab_bytes=0, group_offsets=None, groups=0, c_slab_bytes=0, tile_scale_slab_bytes=0,
                normalize=False, vec_scale=1.0, rope=None, split_slab_bytes=0, segments=(), k_major=False):
        """segments: up to three further products (a_i, b_i, alpha_i, alpha_ptr_i) added into the same C in the same launch;
        k_major: a is [k][m] and b is [k][n] (pass m, n, k)"""
        args = GemmArgs()
        args.a, args.b, args.c = mat(a), mat(b), mat(c)
        args.abType, args.cType = ab_type, c_type
        args.m = a.shape[0] if m is None else m
        args.n = b.shape[0] if n is None else n
        args.tileGroup, args.bSlabBytes = ptr(tile_group), b_slab_bytes
        args.groupOffsets, args.groups, args.cSlabBytes, args.tileScaleSlabBytes = ptr(group_offsets), groups, c_slab_bytes, tile_scale_slab_bytes
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
        args.normalize, args.vecScale, args.rope = int(normalize), vec_scale, mat(rope)
        args.splitSlabBytes = split_slab_bytes
        args.extraSegments = len(segments)
        args.kMajor = int(k_major)
        for i, (sa, sb, sal, sp) in enumerate(segments):
            assert sa.stride(0) == a.stride(0) and sb.stride(0) == b.stride(0)
            args.segment[i].a, args.segment[i].b, args.segment[i].alpha, args.segment[i].alphaPtr = sa.data_ptr(), sb.data_ptr(), sal, ptr(sp)
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


def model_schedule(depth, experts=0, wide_window=64):
    """(layer_type, layer_att_id, layer_slope, att_width) of a model depth: ts2_model_schedule (host only, no GPU needed)"""
    import numpy as np
    lib = load()
    cap = 4 * max(depth, 1) + 8
    lt = np.zeros(cap, np.int32); la = np.zeros(cap, np.int32); ls = np.zeros(cap, np.float32); aw = np.zeros(3, np.int32)
    cnt = C.c_int32(0)
    n = lib.dll.ts2_model_schedule(C.c_int32(depth), C.c_int32(experts), C.c_int32(wide_window), C.c_int32(cap), lt.ctypes.data_as(C.c_void_p),
                                   la.ctypes.data_as(C.c_void_p), ls.ctypes.data_as(C.c_void_p), aw.ctypes.data_as(C.c_void_p), C.byref(cnt))
    if n < 0:
        raise RuntimeError(f"ts2_model_schedule failed with code {n}")
    return lt[:n].copy(), la[:n].copy(), ls[:n].copy(), aw[:cnt.value].copy()


def layer_shapes(ltype, dim, heads, ffn, xp=0, experts=0):
    """[out][in] shapes of a layer's matrices in ts2_model_set_matrix order (EnumLayerMatrices, src/gpt/model_params/model_dim.h:225-262):
    attention Q, K, V, gate, combiner; FFN expand, gate, contract; MoE expand, gate, contract, select"""
    q = heads * 128
    if ltype == 0:
        return [(q, dim), (q, dim), (q, dim), (q, dim), (dim, q)]
    if ltype == 2:
        return [(ffn, dim), (ffn, dim), (dim, ffn)]
    return [(xp * experts, dim), (xp * experts, dim), (dim * experts, xp), (experts, dim)]


def fill_rope_buf(width, rope_len):
    """fp32 [rope_len][width] (cos, sin) table: ts2_fill_rope_buf (host only)"""
    import numpy as np
    lib = load()
    buf = np.zeros((rope_len, width), np.float32)
    lib.check(lib.dll.ts2_fill_rope_buf(buf.ctypes.data_as(C.c_void_p), C.c_int32(width), C.c_int32(rope_len)), "ts2_fill_rope_buf")
    return buf


_probe = None


def _probe_lib():
    global _probe
    if _probe is None:
        if not os.path.exists(PROBE_SO):
            raise RuntimeError(f"{PROBE_SO} is missing: build it with `python -m tscale2_amd.build`")
        _probe = C.CDLL(PROBE_SO)
    return _probe


def probe_mfma_rate(ab_type, random_data, iters=20000):
    """Sustained rate, in T(FL)OP/s, of a kernel that issues nothing but MFMAs of the given operand type on every CU."""
    import torch
    lib = load()
    scratch = torch.empty(1024 * 256, dtype=torch.int32, device="cuda")
    out = C.c_double(0)
    lib.check(_probe_lib().ts2_probe_mfma_rate(C.c_int32(ab_type), C.c_int32(int(random_data)), C.c_int32(iters), ptr(scratch),
                                          C.c_int64(scratch.numel()), C.byref(out), lib.stream()), "ts2_probe_mfma_rate")
    return out.value


def probe_copy_rate(nbytes=1 << 30):
    """Read + write GB/s of a plain 16-byte-per-lane copy of nbytes bytes."""
    import torch
    lib = load()
    src = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    out = C.c_double(0)
    lib.check(_probe_lib().ts2_probe_copy_rate(ptr(src), ptr(dst), C.c_int64(nbytes), C.byref(out), lib.stream()), "ts2_probe_copy_rate")
    return out.value


def probe_shader_clock(run, seconds=0.25, period_us=100):
    """MHz of the shader clock while run() keeps the GPU busy on the current stream: a one-wave monitor kernel on a second stream samples
    the core-clock counter against the 100 MHz counter every period_us; returns (median, min, max) over the samples of the busy time."""
    import torch
    lib = load()
    n = int(seconds * 1e6 / period_us)
    out = torch.zeros(2 * n, dtype=torch.int64, device="cuda")
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        lib.check(_probe_lib().ts2_probe_clock_monitor(ptr(out), C.c_int32(n), C.c_int32(period_us * 100),
                                                       C.c_void_p(side.cuda_stream)), "ts2_probe_clock_monitor")
    e0 = torch.cuda.Event(enable_timing=True); e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    run()
    e1.record()
    torch.cuda.synchronize()
    busy_ms = e0.elapsed_time(e1)
    v = out.view(n, 2).double().cpu()
    mhz = (v[:, 1] / v[:, 0] * 100.0)
    k = max(1, min(n, int(busy_ms * 1e3 / period_us)))      # samples taken while run() was executing
    body = mhz[k // 10: max(k // 10 + 1, k - k // 10)]       # (without the ramp at either end)
    return float(body.median()), float(body.min()), float(body.max())


class BwdBuffers(C.Structure):
    _fields_ = [("grad8", Mat), ("grad8RowScale", C.c_void_p), ("gradT", Mat), ("srcT", Mat), ("tileMax", C.c_void_p), ("tileScale", C.c_void_p),
                ("transformT", Mat), ("partial", Mat), ("splits", C.c_int32), ("gradRowAbsMax", C.c_void_p),
                ("gradRowAbsMaxValid", C.c_int32), ("srcTValid", C.c_int32), ("gradTValid", C.c_int32), ("transformTValid", C.c_int32),
                ("rowOrder", C.c_void_p), ("rowOrderTmp", C.c_void_p), ("sortRows", C.c_int32), ("padRowsZero", C.c_int32),
                ("ditherSeed", C.c_uint32)]


class MatMulBuffers:
    """Scratch of one linear layer's backward, allocated with torch (the reference allocates the same members from its pools,
    src/gpt/compute/matmul_fwdbwd.cuh:283-311).  mode: I8 or E4M3."""

    def __init__(self, mode, len_round, src_dim, grad_dim, k_tile=512, splits=1, share_row_max=False, sort_rows=False):
        import torch
        self.mode, self.len_round, self.src_dim, self.grad_dim, self.k_tile = mode, len_round, src_dim, grad_dim, k_tile
        bt = torch.int8 if mode == I8 else torch.uint8
        dev = "cuda"
        self.t = {}
        if mode == I8:
            self.t["grad8"] = torch.empty((len_round, grad_dim), dtype=torch.int8, device=dev)
            self.t["grad8RowScale"] = torch.empty(len_round, dtype=torch.float32, device=dev)
            n_tiles = len_round // k_tile
            self.t["tileMax"] = torch.empty(n_tiles, dtype=torch.float32, device=dev)
            self.t["tileScale"] = torch.empty(n_tiles, dtype=torch.float32, device=dev)
        self.t["gradT"] = torch.empty((grad_dim, len_round), dtype=bt, device=dev)
        self.t["srcT"] = torch.empty((src_dim, len_round), dtype=bt, device=dev)
        self.t["transformT"] = torch.empty((src_dim, grad_dim), dtype=bt, device=dev)
        self.c = BwdBuffers()
        for k, v in self.t.items():
            setattr(self.c, k, mat(v) if v.dim() == 2 else v.data_ptr())
        if share_row_max and mode == I8:
            # backprop_multi and backprop_delta will be given the same gradient tensor: the delta reuses the row maxima of the first
            self.t["gradRowAbsMax"] = torch.empty(len_round, dtype=torch.float32, device=dev)
            self.c.gradRowAbsMax = self.t["gradRowAbsMax"].data_ptr()
            self.c.gradRowAbsMaxValid = 1
        if sort_rows:
            assert share_row_max and mode == I8, "the sorted delta needs the row maxima that backprop_multi leaves"
            self.t["rowOrder"] = torch.empty(len_round, dtype=torch.int32, device=dev)
            self.t["rowOrderTmp"] = torch.empty(len_round, dtype=torch.int32, device=dev)
            self.c.rowOrder, self.c.rowOrderTmp, self.c.sortRows = self.t["rowOrder"].data_ptr(), self.t["rowOrderTmp"].data_ptr(), 1
        if splits > 1:
            self.t["partial"] = torch.empty((splits * grad_dim, src_dim), dtype=torch.float32, device=dev)
            self.c.partial = mat(self.t["partial"])
            self.c.splits = splits
        self.delta = torch.empty((grad_dim, src_dim), dtype=torch.int8, device=dev)
        self.delta_tile_scale = torch.empty((src_dim // 128, grad_dim), dtype=torch.float32, device=dev)

    def backprop_multi(self, len_, transform_fast, grad, grad_type, grad_col_scale=None):
        call("ts2_matmul_backprop_multi", self.mode, len_, self.len_round, self.src_dim, self.grad_dim, transform_fast, grad, grad_type,
             grad_col_scale, C.byref(self.c))

    def backprop(self, len_, grad, alpha, alpha_ptr, src_grad, src_grad_type, add=False):
        call("ts2_matmul_backprop", self.mode, len_, self.len_round, self.src_dim, self.grad_dim, grad, C.byref(self.c), float(alpha), alpha_ptr,
             src_grad, src_grad_type, int(add))

    def backprop_delta(self, len_, src, src_row_scale, grad, grad_type, grad_scale=None, alpha=1.0):
        call("ts2_matmul_backprop_delta", self.mode, len_, self.len_round, self.src_dim, self.grad_dim, src, src_row_scale, grad, grad_type,
             float(alpha), grad_scale, self.k_tile, C.byref(self.c), self.delta, self.delta_tile_scale)

    def delta_fp32(self):
        """dequantised packed delta [gradDim][srcDim]"""
        sc = self.delta_tile_scale.t().repeat_interleave(128, dim=1)
        return self.delta.float() * sc


def matmul_backprop_group(bufs, len_, grads, alphas, alpha_ptrs, src_grad, src_grad_type, add=False, check=True):
    """ts2_matmul_backprop_group over MatMulBuffers objects of equal shape whose backprop_multi has run: src_grad (+)= sum of the products"""
    lib = load()
    n = len(bufs)
    b0 = bufs[0]
    gm = [mat(g) if g is not None else Mat(None, 0, 0, 0) for g in grads]
    gp = (C.POINTER(Mat) * n)(*[C.pointer(m) for m in gm])
    bp = (C.POINTER(BwdBuffers) * n)(*[C.pointer(b.c) for b in bufs])
    al = (C.c_float * n)(*[float(a) for a in alphas])
    ap = (C.c_void_p * n)(*[None if p is None else p.data_ptr() for p in alpha_ptrs])
    sg = mat(src_grad)
    rc = lib.dll.ts2_matmul_backprop_group(C.c_int32(b0.mode), C.c_int32(len_), C.c_int32(b0.len_round), C.c_int32(b0.src_dim), C.c_int32(b0.grad_dim),
                                           C.c_int32(n), gp, bp, al, ap, C.byref(sg), C.c_int32(src_grad_type), C.c_int32(int(add)), lib.stream())
    if check:
        lib.check(rc, "ts2_matmul_backprop_group")
    return rc


class AttArgs(C.Structure):
    _fields_ = [("len", C.c_int32), ("lenRound", C.c_int32), ("heads", C.c_int32), ("q", Mat), ("k", Mat), ("v", Mat),
                ("spanStart", C.c_void_p), ("spanFinish", C.c_void_p), ("attDotScale", C.c_float), ("alibiSlope", C.c_float),
                ("valLookup", Mat), ("sumWeightLog", Mat)]


class AttGradArgs(C.Structure):
    _fields_ = [("len", C.c_int32), ("lenRound", C.c_int32), ("heads", C.c_int32), ("q", Mat), ("k", Mat), ("v", Mat), ("dValLookup", Mat),
                ("spanStart", C.c_void_p), ("spanFinish", C.c_void_p), ("revLo", C.c_void_p), ("revHi", C.c_void_p),
                ("attDotScale", C.c_float), ("alibiSlope", C.c_float), ("sumWeightLog", Mat), ("dScale", Mat), ("dQ", Mat), ("dK", Mat),
                ("dV", Mat), ("gradType", C.c_int32), ("which", C.c_int32), ("dsBase", C.c_void_p), ("dsScratch", C.c_void_p),
                ("dsCapacityBlocks", C.c_int64)]


def att_forward(len_, heads, q, k, v, span_start, span_finish, att_dot_scale, slope, val_lookup, sum_weight_log):
    a = AttArgs(len_, q.shape[0], heads, mat(q), mat(k), mat(v), span_start.data_ptr(), span_finish.data_ptr(), att_dot_scale, slope,
                mat(val_lookup), mat(sum_weight_log))
    lib = load()
    lib.check(lib.dll.ts2_att_forward(C.byref(a), lib.stream()), "ts2_att_forward")


def att_backward(len_, heads, q, k, v, dval, span_start, span_finish, rev_lo, rev_hi, att_dot_scale, slope, sum_weight_log, dscale, dq, dk,
                 dv, grad_type, which=3, ds=None):
    """ds: optional (dsBase, dsScratch) pair - the index of ts2_att_build_ds_index and a uint8 tensor of whole 2048-byte blocks - with which
    dQ is formed from the score gradients the dK/dV kernel leaves behind"""
    a = AttGradArgs(len_, q.shape[0], heads, mat(q), mat(k), mat(v), mat(dval), span_start.data_ptr(), span_finish.data_ptr(),
                    rev_lo.data_ptr(), rev_hi.data_ptr(), att_dot_scale, slope, mat(sum_weight_log), mat(dscale), mat(dq), mat(dk), mat(dv),
                    grad_type, which, None, None, 0)
    if ds is not None:
        a.dsBase, a.dsScratch, a.dsCapacityBlocks = ds[0].data_ptr(), ds[1].data_ptr(), ds[1].numel() // 2048
    lib = load()
    lib.check(lib.dll.ts2_att_backward(C.byref(a), lib.stream()), "ts2_att_backward")


def att_ds_scratch(len_round, heads, span_start, span_finish):
    """(dsBase, dsScratch) for att_backward(ds=...): the block index on the device and an array sized from the host copy of the spans"""
    import torch
    lib = load()
    base = torch.empty(len_round + 1, dtype=torch.int32, device="cuda")
    lib.check(lib.dll.ts2_att_build_ds_index(C.c_int32(len_round), C.c_void_p(span_start.data_ptr()), C.c_void_p(span_finish.data_ptr()),
                                             C.c_void_p(base.data_ptr()), lib.stream()), "ts2_att_build_ds_index")
    hs, hf = span_start.cpu().numpy(), span_finish.cpu().numpy()
    lib.dll.ts2_att_ds_blocks.restype = C.c_int64
    blocks = lib.dll.ts2_att_ds_blocks(C.c_int32(len_round), hs.ctypes.data_as(C.c_void_p), hf.ctypes.data_as(C.c_void_p))
    if blocks < 0:
        raise RuntimeError("ts2_att_ds_blocks failed")
    scratch = torch.empty(max(int(blocks) * heads, 1) * 2048, dtype=torch.uint8, device="cuda")
    return base, scratch


class ModelConfig(C.Structure):
    _fields_ = [("mode", C.c_int32), ("dim", C.c_int32), ("headCount", C.c_int32), ("ffnDim", C.c_int32), ("expertDim", C.c_int32),
                ("expertCount", C.c_int32), ("moeSelected", C.c_int32), ("depth", C.c_int32), ("layerType", C.c_void_p),
                ("layerAttId", C.c_void_p), ("layerSlope", C.c_void_p), ("attTypeCount", C.c_int32), ("vocab", C.c_int32),
                ("labelCount", C.c_int32), ("maxLen", C.c_int32), ("kTile", C.c_int32), ("recompute", C.c_int32), ("ditherSeed", C.c_uint32)]


class AddGradientParams(C.Structure):
    _fields_ = [(n, C.c_float) for n in ("dispDecay", "beta1", "weight0", "weight1", "l2Reg", "stepMult")]


LAYER_EMBED, LAYER_FINAL = -1, -2


class Model:
    """Step driver object of the library (ts2_model_*): owns device buffers, runs forward / backprop of a layer stack."""

    def __init__(self, mode, dim, heads, ffn_dim, layer_type, layer_att_id, layer_slope, att_type_count, vocab, label_count, max_len,
                 expert_dim=0, expert_count=0, moe_selected=0, k_tile=0, recompute=False, dither_seed=0):
        import numpy as np
        self.lib = load()
        dll = self.lib.dll
        dll.ts2_model_create.restype = C.c_void_p
        self._lt = np.ascontiguousarray(layer_type, np.int32)
        self._la = np.ascontiguousarray(layer_att_id, np.int32)
        self._ls = np.ascontiguousarray(layer_slope, np.float32)
        cfg = ModelConfig(mode, dim, heads, ffn_dim, expert_dim, expert_count, moe_selected, len(self._lt), self._lt.ctypes.data,
                          self._la.ctypes.data, self._ls.ctypes.data, att_type_count, vocab, label_count, max_len, k_tile, int(recompute), dither_seed)
        self.h = dll.ts2_model_create(C.byref(cfg))
        if not self.h:
            raise RuntimeError("ts2_model_create failed")
        self.h = C.c_void_p(self.h)
        self.att_type_count = att_type_count

    def close(self):
        if self.h:
            self.lib.dll.ts2_model_destroy(self.h)
            self.h = None

    def _ck(self, rc, what):
        if rc != 0:
            raise RuntimeError(f"{what} failed with code {rc}")

    def set_matrix(self, layer, matrix_id, fast, scale):
        import numpy as np
        fast = np.ascontiguousarray(fast)
        self._ck(self.lib.dll.ts2_model_set_matrix(self.h, layer, matrix_id, fast.ctypes.data_as(C.c_void_p), fast.shape[0], fast.shape[1],
                                                   C.c_float(scale)), "ts2_model_set_matrix")

    def set_master(self, layer, matrix_id, weights, row_disp_size, sparsity=1.0):
        """fp32 master weights of a matrix (optimiser state is created on first use); the fast weights are derived on the device"""
        import numpy as np
        w = np.ascontiguousarray(weights, np.float32)
        self._ck(self.lib.dll.ts2_model_set_master(self.h, layer, matrix_id, w.ctypes.data_as(C.c_void_p), w.shape[0], w.shape[1], row_disp_size,
                                                   C.c_float(sparsity)), "ts2_model_set_master")

    def apply_deltas(self, rate, l2_reg=0.0, beta1=0.0, weight0=1.0, weight1=0.0, disp_decay=0.9):
        """one optimiser step with the deltas of the last backprop (TTrainingStep fields)"""
        p = AddGradientParams(disp_decay, beta1, weight0, weight1, l2_reg, rate)
        self._ck(self.lib.dll.ts2_model_apply_deltas(self.h, C.byref(p), self.lib.stream()), "ts2_model_apply_deltas")

    def get_master(self, layer, matrix_id, rows, cols):
        import numpy as np
        out = np.empty((rows, cols), np.float32)
        self._ck(self.lib.dll.ts2_model_get_master(self.h, layer, matrix_id, out.ctypes.data_as(C.c_void_p), rows, cols), "ts2_model_get_master")
        return out

    def get_matrix(self, layer, matrix_id, rows, cols, dtype):
        """fast weights (bytes of the model's 8-bit type) and the matrix scale"""
        import numpy as np
        out = np.empty((rows, cols), dtype)
        sc = C.c_float(0)
        self._ck(self.lib.dll.ts2_model_get_matrix(self.h, layer, matrix_id, out.ctypes.data_as(C.c_void_p), rows, cols, C.byref(sc)), "ts2_model_get_matrix")
        return out, sc.value

    def set_bias(self, bias):
        import numpy as np
        b = np.ascontiguousarray(bias, np.float32)
        self._ck(self.lib.dll.ts2_model_set_bias(self.h, b.ctypes.data_as(C.c_void_p)), "ts2_model_set_bias")

    def set_batch(self, label_ptr, labels, target_per_row, span_start, span_finish, rope):
        import numpy as np
        lp = np.ascontiguousarray(label_ptr, np.int32); lb = np.ascontiguousarray(labels, np.uint32)
        tg = np.ascontiguousarray(target_per_row, np.int32); rp = np.ascontiguousarray(rope, np.float32)
        ss = [np.ascontiguousarray(a, np.int32) for a in span_start]; sf = [np.ascontiguousarray(a, np.int32) for a in span_finish]
        pa = (C.c_void_p * len(ss))(*[a.ctypes.data for a in ss]); pf = (C.c_void_p * len(sf))(*[a.ctypes.data for a in sf])
        self._ck(self.lib.dll.ts2_model_set_batch(self.h, len(tg), lp.ctypes.data_as(C.c_void_p), lb.ctypes.data_as(C.c_void_p),
                                                  tg.ctypes.data_as(C.c_void_p), pa, pf, rp.ctypes.data_as(C.c_void_p), self.lib.stream()),
                 "ts2_model_set_batch")

    def forward(self):
        self._ck(self.lib.dll.ts2_model_forward(self.h, self.lib.stream()), "ts2_model_forward")

    def backprop(self):
        self._ck(self.lib.dll.ts2_model_backprop(self.h, self.lib.stream()), "ts2_model_backprop")

    def layer_forward(self, layer):
        self._ck(self.lib.dll.ts2_layer_forward(self.h, layer, self.lib.stream()), "ts2_layer_forward")

    def layer_backward(self, layer):
        self._ck(self.lib.dll.ts2_layer_backward(self.h, layer, self.lib.stream()), "ts2_layer_backward")

    def get_delta(self, layer, matrix_id, rows, cols):
        import numpy as np
        out = np.empty((rows, cols), np.float32)
        self._ck(self.lib.dll.ts2_model_get_delta(self.h, layer, matrix_id, out.ctypes.data_as(C.c_void_p), rows, cols), "ts2_model_get_delta")
        return out

    def array(self, name, index=0):
        """torch view (no copy) of an internal device array"""
        import torch
        m = Mat(); t = C.c_int32(0)
        self._ck(self.lib.dll.ts2_model_array(self.h, name.encode(), index, C.byref(m), C.byref(t)), "ts2_model_array")
        dt = {I8: torch.int8, E4M3: torch.uint8, BF16: torch.bfloat16, F32: torch.float32, I32: torch.int32}[t.value]
        es = {I8: 1, E4M3: 1, BF16: 2, F32: 4, I32: 4}[t.value]
        n = m.strideBytes // es * m.y

        class _Holder:
            __cuda_array_interface__ = {"shape": (n,), "typestr": {1: "|u1", 2: "<u2", 4: "<f4"}[es], "data": (m.ptr, False), "version": 2}
        flat = torch.as_tensor(_Holder(), device="cuda")
        if dt == torch.bfloat16:
            flat = flat.view(torch.int16).view(torch.bfloat16)
        elif dt == torch.int8:
            flat = flat.view(torch.int8)
        elif dt == torch.int32:
            flat = flat.view(torch.int32)
        return flat.view(m.y, m.strideBytes // es)[:, :m.x]

    def read(self, name, index=0):
        """host copy (numpy) of an internal device array"""
        import numpy as np
        m = Mat(); t = C.c_int32(0)
        self._ck(self.lib.dll.ts2_model_array(self.h, name.encode(), index, C.byref(m), C.byref(t)), "ts2_model_array")
        dt = {I8: np.int8, E4M3: np.uint8, BF16: np.uint16, F32: np.float32, I32: np.int32}[t.value]
        out = np.empty((m.y, m.x), dt)
        self._ck(self.lib.dll.ts2_model_read(self.h, name.encode(), index, out.ctypes.data_as(C.c_void_p), C.c_int64(out.nbytes)), "ts2_model_read")
        return out

    def loss_sum(self):
        v = C.c_float(0)
        self._ck(self.lib.dll.ts2_model_scalars(self.h, C.byref(v), None, None), "ts2_model_scalars")
        return v.value
