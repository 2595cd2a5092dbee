"""ctypes binding of libbeam_hip.so.

Counterpart of the reference's pybind11 module (python/beam/_C/__init__.py:1-23, signatures in
python/beam/_C/beam_C.pyi:4-23).  Every operator takes (a, b, c): a is [M, K], b is [N, K], c is
[M, N], all 16-bit, all resident on the GPU; c is written in place and nothing is returned.

Tensors may be torch CUDA tensors (launched on torch's current stream) or beam.DeviceArray
objects (memory owned through the library's own allocator, launched on the default stream).
There is no CPU fallback: if the shared library is missing the import fails, and every error
code of the library becomes a BeamError.
"""
from __future__ import annotations

import ctypes
import os
import sys
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np

F16 = 0
BF16 = 1
_DTYPE_NAMES = {F16: "fp16", BF16: "bf16"}

_PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_LIB_PATH = os.path.join(_PKG_DIR, "libbeam_hip.so")


class BeamError(RuntimeError):
    """A call into libbeam_hip.so returned a non-zero status."""

    def __init__(self, status: int, message: str):
        super().__init__(f"beam status {status}: {message}")
        self.status = status


class _TileCfg(ctypes.Structure):
    _fields_ = [("block_m", ctypes.c_int), ("block_n", ctypes.c_int), ("wave_m", ctypes.c_int),
                ("wave_n", ctypes.c_int), ("pipeline", ctypes.c_int), ("group_m", ctypes.c_int)]


class _Problem(ctypes.Structure):
    _fields_ = [("A", ctypes.c_void_p), ("B", ctypes.c_void_p), ("C", ctypes.c_void_p),
                ("gamma", ctypes.c_void_p), ("beta", ctypes.c_void_p), ("eps", ctypes.c_float),
                ("M", ctypes.c_int), ("N", ctypes.c_int), ("K", ctypes.c_int), ("dtype", ctypes.c_int),
                ("split_k", ctypes.c_int), ("ws", ctypes.c_void_p), ("ws_bytes", ctypes.c_size_t),
                ("side_x", ctypes.c_void_p), ("side_y", ctypes.c_void_p), ("side_count", ctypes.c_longlong),
                ("ln_mode", ctypes.c_int)]


def library_path() -> str:
    return _LIB_PATH


def _load() -> ctypes.CDLL:
    if not os.path.exists(_LIB_PATH):
        raise ImportError(
            f"{_LIB_PATH} is missing: build it with `make -C {os.path.join(_PKG_DIR, 'csrc')}` "
            "(hipcc, gfx950).  There is no fallback path.")
    # PyTorch wheels bundle their own HIP runtime.  If torch is imported first, the dynamic linker
    # hands that same runtime to libbeam_hip.so (one runtime per process: tensors and streams can be
    # shared).  Loaded the other way round, torch would bring a second runtime and fail to see the GPU.
    global _TORCH_FIRST
    _TORCH_FIRST = "torch" in sys.modules
    L = ctypes.CDLL(_LIB_PATH)
    vp, i, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    cfgp = ctypes.POINTER(_TileCfg)
    L.beam_last_error.restype = ctypes.c_char_p
    L.beam_init.restype = i
    L.beam_device_info.argtypes = [ctypes.c_char_p, i, ctypes.POINTER(i), ctypes.POINTER(i), ctypes.POINTER(sz)]
    L.beam_num_configs.restype = i
    L.beam_get_config.argtypes = [i, cfgp]
    L.beam_default_config.argtypes = [i, i, i, cfgp, ctypes.POINTER(i)]
    L.beam_gemmrc.argtypes = [vp, vp, vp, i, i, i, i, cfgp, vp]
    for name in ("beam_custom_gemmrc_128x128", "beam_custom_gemmrc_128x256", "beam_custom_gemmrc_256x128"):
        getattr(L, name).argtypes = [vp, vp, vp, i, i, i, vp]
    L.beam_slice_heuristic.argtypes = [i, i]
    L.beam_splitk_workspace_bytes.argtypes = [i, i, i]
    L.beam_splitk_workspace_bytes.restype = sz
    L.beam_gemmrc_splitk.argtypes = [vp, vp, vp, i, i, i, i, cfgp, i, vp, sz, vp]
    L.beam_splitk_effective.argtypes = [i, i, i, cfgp, i]
    L.beam_set_splitk_two_launches.argtypes = [i]
    L.beam_gemmrc_splitk_timed_out.argtypes = [vp, sz, i, i, i, vp, ctypes.POINTER(i)]
    L.beam_splitk_noalloc_max_bytes.argtypes = []
    L.beam_splitk_noalloc_max_bytes.restype = sz
    L.beam_gemmrc_splitk_noalloc.argtypes = [vp, vp, vp, i, i, i, i, cfgp, i, vp]
    L.beam_gemmrc_ln_workspace_bytes.argtypes = [i, i, cfgp]
    L.beam_gemmrc_ln_workspace_bytes.restype = sz
    L.beam_gemmrc_ln.argtypes = [vp, vp, vp, vp, ctypes.c_float, vp, i, i, i, i, cfgp, vp, sz, vp]
    L.beam_gemmrc_ln_workspace_bytes_ex.argtypes = [i, i, cfgp, i]
    L.beam_gemmrc_ln_workspace_bytes_ex.restype = sz
    L.beam_gemmrc_ln_workspace_bytes_for.argtypes = [i, i, i, cfgp, i]
    L.beam_gemmrc_ln_workspace_bytes_for.restype = sz
    L.beam_gemmrc_ln_ex.argtypes = [vp, vp, vp, vp, ctypes.c_float, vp, i, i, i, i, cfgp, i, vp, sz, vp]
    L.beam_gemmrc_ln_checked.argtypes = [vp, vp, vp, vp, ctypes.c_float, vp, i, i, i, i, cfgp, vp, sz, vp, ctypes.POINTER(i)]
    L.beam_set_ln_spin_limit.argtypes = [i]
    L.beam_set_verbose.argtypes = [i]
    L.beam_gemmrc_ln_workspace_reset.argtypes = [vp]
    L.beam_gemmrc_ln_timed_out.argtypes = [vp, vp, ctypes.POINTER(i)]
    L.beam_parallel_gemmrc_silu.argtypes = [vp, vp, vp, i, i, i, vp, vp, ctypes.c_longlong, i, cfgp, vp]
    L.beam_silu.argtypes = [vp, vp, ctypes.c_longlong, i, vp]
    L.beam_matmul_nn.argtypes = [vp, vp, vp, i, i, i, i, cfgp, vp]
    L.beam_bench.argtypes = [i, ctypes.POINTER(_Problem), cfgp, i, i, vp, ctypes.POINTER(ctypes.c_float)]
    L.beam_stream_create.argtypes = [ctypes.POINTER(vp)]
    L.beam_stream_destroy.argtypes = [vp]
    L.beam_graph_begin_capture.argtypes = [vp]
    L.beam_graph_end_capture.argtypes = [vp, ctypes.POINTER(vp)]
    L.beam_graph_launch.argtypes = [vp, vp]
    L.beam_graph_destroy.argtypes = [vp]
    L.beam_event_create.argtypes = [ctypes.POINTER(vp)]
    L.beam_event_record.argtypes = [vp, vp]
    L.beam_event_elapsed_ms.argtypes = [vp, vp, ctypes.POINTER(ctypes.c_float)]
    L.beam_event_destroy.argtypes = [vp]
    L.beam_malloc.argtypes = [ctypes.POINTER(vp), sz]
    L.beam_free.argtypes = [vp]
    L.beam_memcpy_h2d.argtypes = [vp, vp, sz]
    L.beam_memcpy_d2h.argtypes = [vp, vp, sz]
    L.beam_memcpy_d2d.argtypes = [vp, vp, sz]
    L.beam_memset.argtypes = [vp, i, sz]
    L.beam_sync.argtypes = [vp]
    L.beam_host_fill_uniform.argtypes = [vp, sz, i, ctypes.c_uint64, ctypes.c_uint64]
    L.beam_host_fill_normal.argtypes = [vp, sz, i, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_float, ctypes.c_float]
    # test and measurement surface (include/beam_hip_debug.h)
    L.beam_probe_mfma.argtypes = [i, i, i, i, i, i, vp, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_double)]
    L.beam_dbg_ln_plan_bytes.argtypes = [i, i, i, cfgp, i, i, i, i]
    L.beam_dbg_ln_plan_bytes.restype = sz
    L.beam_dbg_assume_compute_units.argtypes = [i]
    L.beam_set_ln_walk.argtypes = [i]
    L.beam_dbg_set_splitk_self_reduce.argtypes = [i]
    L.beam_dbg_tile_of_workgroup.argtypes = [i, i, i, i, ctypes.POINTER(i), ctypes.POINTER(i)]
    L.beam_dbg_lds_offset.argtypes = [i, i]
    L.beam_dbg_kmajor_lds_offset.argtypes = [i, i, i]
    L.beam_dbg_ln_default_config.argtypes = [i, i, i, i, ctypes.POINTER(_TileCfg)]
    L.beam_dbg_w4_kmajor_swizzle.argtypes = [i]
    L.beam_dbg_w4_kmajor_read_offset.argtypes = [i, i, i, i, i]
    L.beam_dbg_band_block_tile.argtypes = [i, i, i, i, i, ctypes.POINTER(i), ctypes.POINTER(i)]
    L.beam_dbg_band_block_grid.argtypes = [i, i, i]
    L.beam_dbg_band_xcd_tile.argtypes = [i, i, i, i, ctypes.POINTER(i), ctypes.POINTER(i)]
    L.beam_dbg_band_xcd_grid.argtypes = [i, i, i]
    L.beam_dbg_band_order_tile.argtypes = [i, i, i, i, i, ctypes.POINTER(i), ctypes.POINTER(i)]
    return L


_TORCH_FIRST = False
lib = _load()


def _check(status: int) -> None:
    if status != 0:
        raise BeamError(status, lib.beam_last_error().decode())


# ---------------------------------------------------------------------------- configurations


@dataclass(frozen=True)
class TileConfig:
    """One point of the tunable space: workgroup tile, wavefront tile, pipeline depth, raster group."""
    block_m: int
    block_n: int
    wave_m: int
    wave_n: int
    pipeline: int = 0
    group_m: int = 0

    def to_c(self) -> _TileCfg:
        return _TileCfg(self.block_m, self.block_n, self.wave_m, self.wave_n, self.pipeline, self.group_m)

    @property
    def name(self) -> str:
        s = f"{self.block_m}x{self.block_n}_w{self.wave_m}x{self.wave_n}"
        if self.pipeline:
            s += {1: "_p22", 2: "_deep"}.get(self.pipeline, f"_p{self.pipeline}")
        if self.group_m:
            s += f"_g{self.group_m}"
        return s


def list_configs() -> List[TileConfig]:
    out = []
    for idx in range(lib.beam_num_configs()):
        c = _TileCfg()
        _check(lib.beam_get_config(idx, ctypes.byref(c)))
        out.append(TileConfig(c.block_m, c.block_n, c.wave_m, c.wave_n, c.pipeline, 0))
    return out


def default_config(M: int, N: int, K: int, split: bool = False):
    """(tile, K slices) the library would use.  split=False: the best tile for a call without a
    workspace (gemmrc), slices = 1; split=True: the best tile together with its slice count
    (gemmrc_splitk)."""
    c = _TileCfg()
    s = ctypes.c_int(1)
    _check(lib.beam_default_config(M, N, K, ctypes.byref(c), ctypes.byref(s) if split else None))
    return TileConfig(c.block_m, c.block_n, c.wave_m, c.wave_n, c.pipeline, c.group_m), s.value


def device_info() -> dict:
    name = ctypes.create_string_buffer(256)
    cus, clk, mem = ctypes.c_int(), ctypes.c_int(), ctypes.c_size_t()
    _check(lib.beam_device_info(name, 256, ctypes.byref(cus), ctypes.byref(clk), ctypes.byref(mem)))
    return {"name": name.value.decode(), "compute_units": cus.value, "clock_khz": clk.value,
            "memory_bytes": mem.value}


# ---------------------------------------------------------------------------- device buffers


class DeviceArray:
    """A 16-bit (or raw byte) buffer in HBM owned through beam_malloc/beam_free."""

    def __init__(self, shape: Sequence[int], dtype: int = F16, itemsize: int = 2):
        self.shape = tuple(int(s) for s in shape)
        self.dtype = dtype
        self.itemsize = itemsize
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * itemsize
        p = ctypes.c_void_p()
        _check(lib.beam_malloc(ctypes.byref(p), self.nbytes))
        self.ptr = p.value or 0

    @classmethod
    def from_numpy(cls, bits: np.ndarray, dtype: int = F16) -> "DeviceArray":
        bits = np.ascontiguousarray(bits)
        arr = cls(bits.shape, dtype, bits.dtype.itemsize)
        _check(lib.beam_memcpy_h2d(arr.ptr, bits.ctypes.data, arr.nbytes))
        return arr

    def to_numpy(self, np_dtype=np.uint16) -> np.ndarray:
        out = np.empty(self.shape, dtype=np_dtype)
        assert out.nbytes == self.nbytes
        _check(lib.beam_sync(None))
        _check(lib.beam_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes))
        return out

    def fill_bytes(self, byte: int = 0) -> None:
        _check(lib.beam_memset(self.ptr, byte, self.nbytes))

    def data_ptr(self) -> int:
        return self.ptr

    def free(self) -> None:
        if getattr(self, "ptr", 0):
            lib.beam_free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _is_torch(x) -> bool:
    return type(x).__module__.split(".")[0] == "torch"


def _describe(x):
    """(pointer, shape, dtype code, stream handle) of a torch tensor or DeviceArray."""
    if isinstance(x, DeviceArray):
        return x.ptr, x.shape, x.dtype, None
    if _is_torch(x):
        if not _TORCH_FIRST:
            raise BeamError(1, "torch tensors need `import torch` before `import beam` (one HIP runtime per "
                               "process); use beam.DeviceArray otherwise")
        import torch
        if not x.is_cuda:
            raise BeamError(1, "tensor is not on the GPU")
        if not x.is_contiguous():
            raise BeamError(1, "tensor is not contiguous")
        if x.dtype == torch.float16:
            d = F16
        elif x.dtype == torch.bfloat16:
            d = BF16
        else:
            raise BeamError(2, f"unsupported tensor type {x.dtype}")
        return x.data_ptr(), tuple(x.shape), d, torch.cuda.current_stream().cuda_stream
    raise TypeError(f"expected a torch CUDA tensor or beam.DeviceArray, got {type(x)!r}")


def _problem(a, b, c):
    """Shape conventions of cuda/cutlass_kernels/main.cc:25-35: M=a.size(0), N=b.size(0),
    K=a.size(1); a.size(1)==b.size(1), c is [M, N]; all three of one 16-bit dtype."""
    pa, sa, da, st = _describe(a)
    pb, sb, db, _ = _describe(b)
    pc, sc, dc, _ = _describe(c)
    if len(sa) != 2 or len(sb) != 2 or len(sc) != 2:
        raise BeamError(1, "a, b, c must be 2-D")
    M, K = sa
    N = sb[0]
    if sb[1] != K:
        raise BeamError(1, f"a.size(1)={K} != b.size(1)={sb[1]}")
    if sc != (M, N):
        raise BeamError(1, f"c has shape {sc}, expected {(M, N)}")
    if not (da == db == dc):
        raise BeamError(2, "a, b, c must share one dtype (fp16 or bf16)")
    return pa, pb, pc, M, N, K, da, st


def _cfg_from_shapes(shape_threadblock, shape_warp, pipeline=0, group_m=0) -> _TileCfg:
    # An empty list means "default", as in cuda/cutlass_kernels/cutlass_gemmrc.cu:73-81.
    tb = list(shape_threadblock) if shape_threadblock else [128, 128]
    wp = list(shape_warp) if shape_warp else [64, 64]
    if len(tb) != 2 or len(wp) != 2:
        raise BeamError(1, "shape_threadblock and shape_warp must have two entries")
    return _TileCfg(tb[0], tb[1], wp[0], wp[1], pipeline, group_m)


# ---------------------------------------------------------------------------- workspaces

_workspace: Optional[DeviceArray] = None
_ln_workspace: Optional[DeviceArray] = None  # fused GEMM+LayerNorm keeps state in its workspace: never shared


def _get_ln_workspace(nbytes: int) -> DeviceArray:
    global _ln_workspace
    if _ln_workspace is None or _ln_workspace.nbytes < nbytes:
        if _ln_workspace is not None:
            _check(lib.beam_sync(None))
            _ln_workspace.free()
        _ln_workspace = DeviceArray((max(nbytes, 1 << 20),), itemsize=1)  # whatever it holds: the library checks
    return _ln_workspace


def _get_workspace(nbytes: int) -> DeviceArray:
    """Grow-only scratch owned by the Python layer (the C ABI itself keeps no hidden buffer);
    counterpart of get_the_buffer, cuda/cutlass_kernels/cutlass_gemmrc_splitk.cu:31-42."""
    global _workspace
    if _workspace is None or _workspace.nbytes < nbytes:
        if _workspace is not None:
            _check(lib.beam_sync(None))
            _workspace.free()
        _workspace = DeviceArray((max(nbytes, 1 << 20),), itemsize=1)
    return _workspace


# ---------------------------------------------------------------------------- operators


def gemmrc(a, b, c, config: Optional[TileConfig] = None) -> None:
    """c = a @ b.T with the library's default tile (or `config`)."""
    pa, pb, pc, M, N, K, d, st = _problem(a, b, c)
    cfg = ctypes.byref(config.to_c()) if config is not None else None
    _check(lib.beam_gemmrc(pa, pb, pc, M, N, K, d, cfg, st))


def gemmrc_spec(a, b, c, shape_threadblock=(128, 128), shape_warp=(64, 64), pipeline: int = 0,
                group_m: int = 0) -> None:
    """c = a @ b.T with an explicit workgroup tile / wavefront tile
    (reference: cutlass_gemmrc_spec, python/beam/_C/beam_C.pyi:16)."""
    pa, pb, pc, M, N, K, d, st = _problem(a, b, c)
    cfg = _cfg_from_shapes(shape_threadblock, shape_warp, pipeline, group_m)
    _check(lib.beam_gemmrc(pa, pb, pc, M, N, K, d, ctypes.byref(cfg), st))


def _splitk(a, b, c, cfgp, split_k_slices: int, check: bool = False) -> None:
    pa, pb, pc, M, N, K, d, st = _problem(a, b, c)
    s = lib.beam_splitk_effective(M, N, K, cfgp, split_k_slices)
    if s < 0:
        raise BeamError(2, lib.beam_last_error().decode())
    need = lib.beam_splitk_workspace_bytes(M, N, s) if s > 1 else 0
    ws = _get_workspace(need) if need else None
    _check(lib.beam_gemmrc_splitk(pa, pb, pc, M, N, K, d, cfgp, split_k_slices,
                                  ws.ptr if ws else None, ws.nbytes if ws else 0, st))
    if check and ws is not None:
        flag = ctypes.c_int(0)
        _check(lib.beam_gemmrc_splitk_timed_out(ws.ptr, ws.nbytes, M, N, s, st, ctypes.byref(flag)))
        if flag.value:
            raise BeamError(4, "split-K: a reducing workgroup gave up waiting for the slices of its tile; "
                               "the outputs concerned are NaN")


def set_splitk_two_launches(on: bool) -> None:
    """True: split-K always runs as partial kernel + reduce kernel; False (default): one launch where it applies."""
    _check(lib.beam_set_splitk_two_launches(1 if on else 0))


def set_ln_walk(on: bool) -> None:
    """True (default): from more 256 x 256 tiles than CUs on, the fused GEMM+LayerNorm of the 4-wavefront kernel runs
    one workgroup per CU walking its tiles (every workgroup of the launch must then be resident at once); False: one
    workgroup per tile in band order, which finishes band by band on whatever share of the device it gets.  Same bits."""
    _check(lib.beam_set_ln_walk(1 if on else 0))


def gemmrc_splitk(a, b, c, split_k_slices: int = 0, check: bool = False) -> None:
    """Split-K with the library's default tile for the problem; split_k_slices <= 0: the library
    picks the slice count as well (one full round of workgroups)
    (reference: cutlass_gemmrc_splitk, python/beam/_C/beam_C.pyi:18).  check=True waits for the
    result and raises if the one-launch form's bounded wait ran out."""
    _splitk(a, b, c, None, split_k_slices, check)


def gemmrc_splitk_spec(a, b, c, shape_threadblock=(128, 128), shape_warp=(64, 64), split_k_slices: int = 0,
                       pipeline: int = 0, group_m: int = 0, check: bool = False) -> None:
    """Split-K with explicit tiles (reference: cutlass_gemmrc_splitk_spec, beam_C.pyi:20)."""
    cfg = _cfg_from_shapes(shape_threadblock, shape_warp, pipeline, group_m)
    _splitk(a, b, c, ctypes.byref(cfg), split_k_slices, check)


LN_AUTO, LN_TWOPASS, LN_FUSED = 0, 1, 2
# the library's default bound on the waits of its kernels (beam_set_ln_spin_limit), for code that changes and restores it
DEFAULT_SPIN_LIMIT = 16384


def gemmrc_ln(a, b, c, gamma, beta, eps: float = 1e-5, config: Optional[TileConfig] = None,
              mode: int = LN_AUTO, check: bool = True) -> bool:
    """c = LayerNorm_N(a @ b.T) * gamma + beta, statistics from the fp32 accumulators.
    mode: LN_AUTO (one kernel when N / block_n <= 64 on a 256-CU device, else two passes), LN_TWOPASS, LN_FUSED.
    check (the default): wait for the result.  The workgroups of the one-kernel form wait for one another, boundedly,
    which assumes that they have the device to themselves; when other work keeps the device occupied and that wait
    runs out, LN_AUTO repeats the call as two passes (the return value is then True, and c is right either way) and
    an explicit LN_FUSED raises BeamError.  check=False launches and returns at once, like the other operators: the
    rows concerned are NaN if that ever happens, and gemmrc_ln_timed_out() tells."""
    pa, pb, pc, M, N, K, d, st = _problem(a, b, c)
    pg, sg, dg, _ = _describe(gamma)
    pbt, sbt, dbt, _ = _describe(beta)
    if tuple(sg) != (N,) or tuple(sbt) != (N,) or dg != d or dbt != d:
        raise BeamError(1, "gamma and beta must be [N] of the same dtype as a, b, c")
    cfg = config.to_c() if config is not None else None
    cfgp = ctypes.byref(cfg) if cfg else None
    # operands aligned to an element only run on the plain kernels, which need room for an fp32 copy of the product
    aligned = ((pa | pb | pc) & 15) == 0 and ((pg | pbt) & 7) == 0
    need = lib.beam_gemmrc_ln_workspace_bytes_for(M, N, K, cfgp, mode) if aligned else lib.beam_gemmrc_ln_workspace_bytes_ex(M, N, cfgp, mode)
    ws = _get_ln_workspace(need)
    if check and mode == LN_AUTO:
        fell_back = ctypes.c_int(0)
        _check(lib.beam_gemmrc_ln_checked(pa, pb, pg, pbt, eps, pc, M, N, K, d, cfgp, ws.ptr, ws.nbytes, st, ctypes.byref(fell_back)))
        return bool(fell_back.value)
    _check(lib.beam_gemmrc_ln_ex(pa, pb, pg, pbt, eps, pc, M, N, K, d, cfgp, mode, ws.ptr, ws.nbytes, st))
    if check:
        flag = ctypes.c_int(0)
        _check(lib.beam_gemmrc_ln_timed_out(ws.ptr, st, ctypes.byref(flag)))
        if flag.value:
            raise BeamError(4, "fused GEMM+LayerNorm gave up waiting for a band of workgroups (device shared with "
                               "other work?); use mode=LN_AUTO or LN_TWOPASS")
    return False


def gemmrc_ln_timed_out() -> bool:
    """True if the last fused GEMM+LayerNorm on the shared workspace gave up waiting for a band."""
    if _ln_workspace is None:
        return False
    flag = ctypes.c_int(0)
    _check(lib.beam_gemmrc_ln_timed_out(_ln_workspace.ptr, None, ctypes.byref(flag)))
    return bool(flag.value)


def matmul(a, b, c=None, config: Optional[TileConfig] = None):
    """c = a @ b with a [M, K] and b [K, N], both row-major; returns c (allocated like the inputs when
    not given).  Reference: matmul(a, b) of python/beam/triton_kernels/gemm.py:78-99."""
    pa, sa, da, st = _describe(a)
    pb, sb, db, _ = _describe(b)
    if len(sa) != 2 or len(sb) != 2 or sa[1] != sb[0]:
        raise BeamError(1, "Incompatible dimensions")
    if da != db:
        raise BeamError(2, "a and b must share one dtype (fp16 or bf16)")
    M, K = sa
    N = sb[1]
    if c is None:
        if _is_torch(a):
            import torch
            c = torch.empty((M, N), device=a.device, dtype=a.dtype)
        else:
            c = DeviceArray((M, N), da)
    pc, sc, dc, _ = _describe(c)
    if tuple(sc) != (M, N) or dc != da:
        raise BeamError(1, f"c must be {(M, N)} of the inputs' dtype")
    cfg = config.to_c() if config is not None else None
    _check(lib.beam_matmul_nn(pa, pb, pc, M, N, K, da, ctypes.byref(cfg) if cfg else None, st))
    return c


def _flat_pair(x, y, d=None):
    px, sx, dx, st = _describe(x)
    py, sy, dy, _ = _describe(y)
    nx, ny = int(np.prod(sx, dtype=np.int64)), int(np.prod(sy, dtype=np.int64))
    if nx != ny:
        raise BeamError(1, f"elementwise input has {nx} elements, output {ny}")
    if dx != dy or (d is not None and dx != d):
        raise BeamError(2, "elementwise input and output must share the GEMM's dtype")
    return px, py, nx, dx, st


def silu(x, y) -> None:
    """y = x / (1 + exp(-x)) elementwise over arrays of equal size (any shape), one streaming kernel."""
    px, py, n, d, st = _flat_pair(x, y)
    _check(lib.beam_silu(px, py, n, d, st))


def parallel_gemmrc_silu(a, b, c, x, y, config: Optional[TileConfig] = None) -> None:
    """c = a @ b.T and, in the same launch, y = silu(x): the elementwise job is streamed through the
    GEMM's K loop.  Reference: cutlass_parallel_gemmrc_lnr(gemmA, gemmB, gemmC, lnA, lnB),
    cuda/cute_kernels/main.cc:55-76 (python/beam/_C/beam_C.pyi:20)."""
    pa, pb, pc, M, N, K, d, st = _problem(a, b, c)
    px, py, n, _, _ = _flat_pair(x, y, d)
    cfg = config.to_c() if config is not None else None
    _check(lib.beam_parallel_gemmrc_silu(pa, pb, pc, M, N, K, px, py, n, d, ctypes.byref(cfg) if cfg else None, st))


def _fixed(fn_name: str):
    cfn = getattr(lib, fn_name)

    def op(a, b, c) -> None:
        pa, pb, pc, M, N, K, d, st = _problem(a, b, c)
        if d != F16:
            raise BeamError(2, f"{fn_name}: fp16 only")
        _check(cfn(pa, pb, pc, M, N, K, st))

    op.__name__ = fn_name[len("beam_"):]
    op.__doc__ = f"Fixed-tile fp16 gemmrc ({fn_name}); reference: python/beam/_C/beam_C.pyi:8-11."
    return op


custom_gemmrc_128x128 = _fixed("beam_custom_gemmrc_128x128")
custom_gemmrc_128x256 = _fixed("beam_custom_gemmrc_128x256")
custom_gemmrc_256x128 = _fixed("beam_custom_gemmrc_256x128")

# The reference's operator names (python/beam/_C/__init__.py:1-11), kept so that scripts written
# against it run unchanged.  Nothing here involves CUTLASS.
cutlass_gemmrc = gemmrc
cutlass_gemmrc_spec = gemmrc_spec
cutlass_gemmrc_splitk = gemmrc_splitk
cutlass_gemmrc_splitk_spec = gemmrc_splitk_spec
cutlass_parallel_gemmrc_lnr = parallel_gemmrc_silu


# ---------------------------------------------------------------------------- timing / data


OP_GEMM, OP_SPLITK, OP_GEMM_LN, OP_GEMM_SILU, OP_SILU, OP_MATMUL_NN = 0, 1, 2, 3, 4, 5
# launches that measure what the machine allows: an empty kernel, two of them, a split-K launch with only its loads
OP_PROBE_EMPTY, OP_PROBE_EMPTY_PAIR, OP_PROBE_SPLITK_LOADS = 6, 7, 8
OP_PROBE_LN_APPLY = 9  # the normalisation pass of a two-pass GEMM+LayerNorm alone (after such a call on the shared workspace)


def bench(op: int, a, b, c, config: Optional[TileConfig] = None, split_k: int = 0, gamma=None, beta=None,
          eps: float = 1e-5, warmup: int = 5, iters: int = 20, x=None, y=None, ln_mode: int = 0) -> float:
    """Average milliseconds per call (HIP events around `iters` back-to-back launches)."""
    if op == OP_MATMUL_NN:  # b is [K, N]
        pa, (M, K), d, st = _describe(a)
        pb, (kb, N), _, _ = _describe(b)
        pc = _describe(c)[0]
        if kb != K or tuple(_describe(c)[1]) != (M, N):
            raise BeamError(1, "Incompatible dimensions")
    else:
        pa, pb, pc, M, N, K, d, st = _problem(a, b, c)
    cfg = config.to_c() if config is not None else None
    cfgp = ctypes.byref(cfg) if cfg is not None else None
    q = _Problem(pa, pb, pc, None, None, eps, M, N, K, d, split_k, None, 0, None, None, 0, ln_mode)
    if op in (OP_GEMM_SILU, OP_SILU):
        q.side_x, q.side_y, q.side_count, _, _ = _flat_pair(x, y, d)
    ws = None
    if op in (OP_SPLITK, OP_PROBE_SPLITK_LOADS):
        s = lib.beam_splitk_effective(M, N, K, cfgp, split_k)
        if s < 0:
            raise BeamError(2, lib.beam_last_error().decode())
        ws = _get_workspace(max(lib.beam_splitk_workspace_bytes(M, N, s), 1))
    elif op in (OP_GEMM_LN, OP_PROBE_LN_APPLY):
        q.gamma, q.beta = _describe(gamma)[0], _describe(beta)[0]
        ws = _get_ln_workspace(lib.beam_gemmrc_ln_workspace_bytes_for(M, N, K, cfgp, LN_TWOPASS if op == OP_PROBE_LN_APPLY else ln_mode))
    if ws is not None:
        q.ws, q.ws_bytes = ws.ptr, ws.nbytes
    ms = ctypes.c_float()
    _check(lib.beam_bench(op, ctypes.byref(q), cfgp, warmup, iters, st, ctypes.byref(ms)))
    return ms.value


MFMA_16X16X32, MFMA_32X32X16 = 0, 1
PROBE_NORMAL, PROBE_ZEROS = 0, 1


def probe_mfma(dtype: int = F16, mfma_shape: int = MFMA_16X16X32, data: int = PROBE_NORMAL, passes: int = 1600,
               warmup: int = 100, iters: int = 200):
    """(milliseconds per launch, TFLOP/s) of the register-only matrix-core loop: every SIMD of the device issues
    passes x 1024 cycles of MFMAs on operands that sit in registers, no memory instruction at all.  What the
    matrix cores sustain on that data at the clock the power cap allows."""
    ms, flop = ctypes.c_float(), ctypes.c_double()
    _check(lib.beam_probe_mfma(dtype, mfma_shape, data, passes, warmup, iters, None, ctypes.byref(ms), ctypes.byref(flop)))
    return ms.value, flop.value / (ms.value * 1e-3) / 1e12


def do_bench(fn, warmup: int = 5, rep: int = 20, stream=None) -> float:
    """Average milliseconds per call of an arbitrary launcher `fn()` (HIP events on `stream`).
    Host-side launch cost is included when the kernels are shorter than it; prefer bench()
    for the library's own operators."""
    for _ in range(warmup):
        fn()
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    _check(lib.beam_event_create(ctypes.byref(e0)))
    _check(lib.beam_event_create(ctypes.byref(e1)))
    try:
        _check(lib.beam_event_record(e0, stream))
        for _ in range(rep):
            fn()
        _check(lib.beam_event_record(e1, stream))
        ms = ctypes.c_float()
        _check(lib.beam_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
    finally:
        lib.beam_event_destroy(e0)
        lib.beam_event_destroy(e1)
    return ms.value / rep


def host_uniform(shape, dtype: int = F16, seed: int = 0, tensor_id: int = 0) -> np.ndarray:
    """uint16 bit patterns of uniform[-1, 1) values (counter-based, reproducible)."""
    out = np.empty(shape, dtype=np.uint16)
    _check(lib.beam_host_fill_uniform(out.ctypes.data, out.size, dtype, seed, tensor_id))
    return out


def host_normal(shape, dtype: int = F16, seed: int = 0, tensor_id: int = 0, mean: float = 0.0,
                scale: float = 1.0) -> np.ndarray:
    """uint16 bit patterns of mean + scale * N(0, 1) values (counter-based, reproducible)."""
    out = np.empty(shape, dtype=np.uint16)
    _check(lib.beam_host_fill_normal(out.ctypes.data, out.size, dtype, seed, tensor_id, mean, scale))
    return out


def sync() -> None:
    _check(lib.beam_sync(None))
