"""ctypes loader of libsalt_gpu_mi355.so and small host-side conveniences
(device buffers as numpy-in / numpy-out).  No computation happens here: every
call goes through the C ABI declared in include/salt_gpu_mi355.h."""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import numpy as np

LIB_PATH = Path(__file__).resolve().parent / "libsalt_gpu_mi355.so"
vp = C.c_void_p


class Q4Job(C.Structure):
    _fields_ = [("vals", vp), ("scales", vp), ("biases", vp), ("xs", vp), ("ys", vp), ("rows", C.c_int)]


class Fp4Job(C.Structure):
    _fields_ = [("packed", vp), ("scales", vp), ("stored_divisor", C.c_float), ("xs", vp), ("ys", vp),
                ("rows", C.c_int)]


class Cell(C.Structure):
    _fields_ = [("kind", C.c_int), ("views", vp * 8), ("n", C.c_uint32), ("aux", C.c_uint32), ("eps", C.c_float),
                ("scalar", C.c_float)]


class FfnLayerDesc(C.Structure):
    _fields_ = [("hidden", C.c_int), ("dense", C.c_int), ("routed", C.c_int), ("n_experts", C.c_int), ("topk", C.c_int),
                ("eps", C.c_float), ("layer_scalar", C.c_float),
                ("pre_norm", vp), ("pre_norm_2", vp), ("router_scale", vp), ("per_expert_scale", vp),
                ("post_norm_1", vp), ("post_norm_2", vp), ("post_norm", vp),
                ("dense_gate", vp * 3), ("dense_up", vp * 3), ("dense_down", vp * 3), ("router", vp * 3),
                ("pool", vp), ("expert_stride", C.c_size_t)]


CELL_RMSNORM, CELL_TOPK, CELL_RESIDUAL_POSTNORM, CELL_PARALLEL_COMBINE, CELL_SOFTCAP, CELL_ROUTER_INPUT = 1, 2, 3, 4, 5, 6

_lib = None

INCLUDE_DIR = Path(__file__).resolve().parent.parent / "include"


def declared_symbols() -> list[str]:
    """Every function name the public headers declare."""
    import re
    names = []
    for header in sorted(INCLUDE_DIR.glob("*.h")):
        text = re.sub(r"/\*.*?\*/", " ", header.read_text(), flags=re.S)
        names += re.findall(r"\b(salt_(?:gpu|mi355)_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))



def _sig(fn, restype, *argtypes):
    fn.restype = restype
    fn.argtypes = list(argtypes)


def load() -> C.CDLL:
    """Loads the shared library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(f"{LIB_PATH} is missing: build it with `make -C salt-core_amd/csrc` "
                           "(or __graft_entry__.build())")
    lib = C.CDLL(str(LIB_PATH))
    i, sz, f = C.c_int, C.c_size_t, C.c_float
    _sig(lib.salt_mi355_init, i)
    _sig(lib.salt_mi355_shutdown, i)
    _sig(lib.salt_mi355_last_error, C.c_char_p)
    _sig(lib.salt_mi355_last_kernel, C.c_char_p)
    _sig(lib.salt_mi355_converter_tables, i, vp, vp)
    _sig(lib.salt_mi355_dev_alloc, vp, sz)
    _sig(lib.salt_mi355_dev_free, i, vp)
    _sig(lib.salt_mi355_dev_upload, i, vp, vp, sz)
    _sig(lib.salt_mi355_dev_download, i, vp, vp, sz)
    _sig(lib.salt_mi355_dev_fill, i, vp, i, sz)
    _sig(lib.salt_mi355_stream, vp)
    _sig(lib.salt_mi355_stream_sync, i, vp)
    _sig(lib.salt_mi355_graph_begin, i, vp)
    _sig(lib.salt_mi355_graph_end, vp, vp)
    _sig(lib.salt_mi355_graph_launch, i, vp, vp)
    _sig(lib.salt_mi355_graph_destroy, i, vp)
    _sig(lib.salt_mi355_set_tolerance_class, i, i)
    _sig(lib.salt_mi355_launch_skeleton_dev, i, i, i, i, i, i, i, vp)
    _sig(lib.salt_mi355_event_create, vp)
    _sig(lib.salt_mi355_event_destroy, i, vp)
    _sig(lib.salt_mi355_event_record, i, vp, vp)
    _sig(lib.salt_mi355_event_elapsed_ms, i, vp, vp, C.POINTER(f))
    _sig(lib.salt_mi355_q4_matvec_dev, i, vp, vp, vp, i, i, i, vp, vp, i, vp)
    _sig(lib.salt_mi355_q4_jobs_dev, i, C.POINTER(Q4Job), i, i, i, i, vp)
    _sig(lib.salt_mi355_q4_matvec_t_dev, i, vp, vp, vp, i, i, i, vp, vp, vp)
    _sig(lib.salt_mi355_q4_jobs_t_dev, i, C.POINTER(Q4Job), i, i, i, vp)
    _sig(lib.salt_mi355_q4_jobs_activated_dev, i, C.POINTER(Q4Job), i, i, C.c_longlong, vp)
    _sig(lib.salt_mi355_q4_matmul_workspace_bytes, sz, i, i)
    _sig(lib.salt_mi355_q4_matmul_dev, i, vp, vp, vp, i, i, i, vp, vp, vp, vp)
    _sig(lib.salt_mi355_nvfp4_qdq_dev, i, vp, i, i, f, vp, vp, vp, vp, vp)
    _sig(lib.salt_mi355_nvfp4_matvec_dev, i, vp, vp, f, i, i, i, vp, vp, i, vp)
    _sig(lib.salt_mi355_nvfp4_jobs_dev, i, C.POINTER(Fp4Job), i, i, i, i, vp)
    _sig(lib.salt_mi355_nvfp4_matvec_qdq_dev, i, vp, vp, f, f, i, i, vp, vp, vp, i, vp)
    _sig(lib.salt_mi355_nvfp4_matvec_t_dev, i, vp, vp, f, f, i, i, i, vp, vp, vp, vp)
    _sig(lib.salt_mi355_nvfp4_jobs_t_dev, i, C.POINTER(Fp4Job), i, i, i, f, vp, vp)
    _sig(lib.salt_mi355_nvfp4_matmul_workspace_bytes, sz, i, i, i)
    _sig(lib.salt_mi355_nvfp4_matmul_dev, i, vp, vp, f, f, i, i, i, vp, vp, vp, vp, vp)
    _sig(lib.salt_mi355_q4_decode_dev, i, vp, vp, vp, sz, vp, vp)
    _sig(lib.salt_mi355_nvfp4_dequant_weights_dev, i, vp, vp, f, i, i, vp, vp)
    _sig(lib.salt_mi355_router_fixture_dev, i, i, i, C.c_uint64, i, C.c_double, vp, vp, vp)
    _sig(lib.salt_mi355_bf16_matvec_dev, i, vp, i, i, i, vp, vp, vp, vp)
    _sig(lib.salt_mi355_q8_matvec_dev, i, vp, vp, vp, i, i, i, vp, vp, vp)
    _sig(lib.salt_mi355_cells_dev, i, C.POINTER(Cell), i, vp, vp)
    _sig(lib.salt_mi355_ffn_block_workspace_bytes, sz, C.POINTER(FfnLayerDesc))
    _sig(lib.salt_mi355_ffn_block_dev, i, C.POINTER(FfnLayerDesc), vp, vp, vp, vp, vp, vp, vp)
    _sig(lib.salt_mi355_router_topk_dev, i, vp, vp, i, i, i, vp, vp, vp, vp)
    _sig(lib.salt_mi355_moe_workspace_bytes, sz, i, i, i, i)
    _sig(lib.salt_mi355_moe_decode_step_dev, i, vp, sz, i, i, i, i, vp, vp, vp, vp, vp, vp, vp, vp, vp)
    _sig(lib.salt_mi355_moe_decode_step_t_dev, i, vp, sz, i, i, i, i, vp, vp, vp, vp, vp, vp, vp, vp, vp)
    _sig(lib.salt_mi355_moe_decode_step_static_dev, i, vp, sz, i, i, i, i, vp, vp, vp, vp, vp, vp, vp, vp, vp)
    _sig(lib.salt_mi355_moe_prefill_workspace_bytes, sz, i, i, i, i, i)
    _sig(lib.salt_mi355_moe_prefill_dev, i, vp, sz, i, i, i, i, i, vp, vp, vp, vp, vp, vp, vp, vp, vp)
    _sig(lib.salt_mi355_moe_activate_dev, i, vp, vp, vp, sz, vp)
    _sig(lib.salt_mi355_moe_reduce_dev, i, vp, vp, i, i, vp, vp)
    _lib = lib
    return lib


def init() -> C.CDLL:
    """Loads the library and initialises the device; raises with the library's
    own message when there is no usable MI355X."""
    lib = load()
    if lib.salt_mi355_init() != 0:
        raise RuntimeError("salt_mi355_init failed: " + lib.salt_mi355_last_error().decode())
    return lib


def check(rc: int, what: str = "call"):
    if rc != 0:
        raise RuntimeError(f"{what} failed: " + load().salt_mi355_last_error().decode())


class DeviceBuffer:
    """A hipMalloc'd region owned by this object."""

    def __init__(self, nbytes: int, fill: int | None = None):
        self.lib = load()
        self.nbytes = int(nbytes)
        self.ptr = self.lib.salt_mi355_dev_alloc(max(self.nbytes, 1))
        if not self.ptr:
            raise MemoryError("salt_mi355_dev_alloc: " + self.lib.salt_mi355_last_error().decode())
        if fill is not None:
            check(self.lib.salt_mi355_dev_fill(self.ptr, fill, self.nbytes), "fill")

    @classmethod
    def from_host(cls, array: np.ndarray) -> "DeviceBuffer":
        array = np.ascontiguousarray(array)
        buf = cls(array.nbytes)
        check(buf.lib.salt_mi355_dev_upload(buf.ptr, array.ctypes.data_as(vp), array.nbytes), "upload")
        return buf

    def upload(self, array: np.ndarray, offset: int = 0):
        array = np.ascontiguousarray(array)
        assert offset + array.nbytes <= self.nbytes
        check(self.lib.salt_mi355_dev_upload(self.ptr + offset, array.ctypes.data_as(vp), array.nbytes), "upload")

    def to_host(self, dtype, count: int | None = None, offset: int = 0) -> np.ndarray:
        dtype = np.dtype(dtype)
        count = (self.nbytes - offset) // dtype.itemsize if count is None else count
        out = np.empty(count, dtype)
        check(self.lib.salt_mi355_dev_download(out.ctypes.data_as(vp), self.ptr + offset, out.nbytes), "download")
        return out

    def at(self, offset: int) -> int:
        return self.ptr + offset

    def free(self):
        if self.ptr:
            self.lib.salt_mi355_dev_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def q4_matvec(vals: np.ndarray, scales: np.ndarray, biases: np.ndarray | None, R: int, C_: int,
              xs: np.ndarray, chains: int = 0, value_offset: int = 0, tolerance_class: bool = False) -> np.ndarray:
    """Host-array convenience around salt_mi355_q4_matvec_dev (or, with tolerance_class, salt_mi355_q4_matvec_t_dev):
    uploads, runs on the library stream, downloads ys[B, R].  value_offset shifts the packed values by that many bytes
    inside their device allocation (alignment cases)."""
    lib = init()
    xs = np.ascontiguousarray(xs, np.float32).reshape(-1, C_)
    B = xs.shape[0]
    dv, ds = DeviceBuffer(vals.nbytes + value_offset + 16, fill=0), DeviceBuffer.from_host(scales)
    dv.upload(vals, value_offset)
    db = DeviceBuffer.from_host(biases) if biases is not None else None
    dx = DeviceBuffer.from_host(xs)
    dy = DeviceBuffer(B * R * 4, fill=0xFF)
    stream = lib.salt_mi355_stream()
    if tolerance_class:
        check(lib.salt_mi355_q4_matvec_t_dev(dv.at(value_offset), ds.ptr, db.ptr if db else None, R, C_, B, dx.ptr,
                                             dy.ptr, stream), "q4_matvec_t_dev")
    else:
        check(lib.salt_mi355_q4_matvec_dev(dv.at(value_offset), ds.ptr, db.ptr if db else None, R, C_, B, dx.ptr, dy.ptr,
                                           chains, stream), "q4_matvec_dev")
    check(lib.salt_mi355_stream_sync(stream), "sync")
    return dy.to_host(np.float32).reshape(B, R)


def nvfp4_qdq(x: np.ndarray, g: float):
    """Host-array convenience around salt_mi355_nvfp4_qdq_dev.  Returns
    (status, packed, scales, dequant)."""
    lib = init()
    x = np.ascontiguousarray(x, np.float32)
    B, C_ = (1, x.shape[0]) if x.ndim == 1 else x.shape
    dx = DeviceBuffer.from_host(x)
    dp, ds, dd = DeviceBuffer(B * C_ // 2, fill=0), DeviceBuffer(B * C_ // 16, fill=0), DeviceBuffer(B * C_ * 4, fill=0)
    st = DeviceBuffer(4, fill=0)
    stream = lib.salt_mi355_stream()
    check(lib.salt_mi355_nvfp4_qdq_dev(dx.ptr, C_, B, g, dp.ptr, ds.ptr, dd.ptr, st.ptr, stream), "nvfp4_qdq_dev")
    check(lib.salt_mi355_stream_sync(stream), "sync")
    return (int(st.to_host(np.int32)[0]), dp.to_host(np.uint8), ds.to_host(np.uint8),
            dd.to_host(np.float32).reshape(x.shape))


def nvfp4_matvec(packed: np.ndarray, scales: np.ndarray, divisor: float, R: int, C_: int, xs: np.ndarray,
                 input_global_scale: float | None = 64.0, chains: int = 0):
    """The reference matvec: activation Q/DQ (skipped when input_global_scale
    is None) followed by the rows.  Returns (status, ys[B, R])."""
    lib = init()
    xs = np.ascontiguousarray(xs, np.float32).reshape(-1, C_)
    B = xs.shape[0]
    dw, ds, dx = DeviceBuffer.from_host(packed), DeviceBuffer.from_host(scales), DeviceBuffer.from_host(xs)
    dq = DeviceBuffer(B * C_ * 4)
    dy = DeviceBuffer(B * R * 4, fill=0xFF)
    st = DeviceBuffer(4, fill=0)
    stream = lib.salt_mi355_stream()
    src = dx
    if input_global_scale is not None:
        check(lib.salt_mi355_nvfp4_qdq_dev(dx.ptr, C_, B, input_global_scale, None, None, dq.ptr, st.ptr, stream),
              "nvfp4_qdq_dev")
        src = dq
    check(lib.salt_mi355_nvfp4_matvec_dev(dw.ptr, ds.ptr, divisor, R, C_, B, src.ptr, dy.ptr, chains, stream),
          "nvfp4_matvec_dev")
    check(lib.salt_mi355_stream_sync(stream), "sync")
    return int(st.to_host(np.int32)[0]), dy.to_host(np.float32).reshape(B, R)


def nvfp4_matvec_t(packed: np.ndarray, scales: np.ndarray, divisor: float, R: int, C_: int, xs: np.ndarray,
                   input_global_scale: float = 64.0):
    """The reference matvec on the tolerance-class kernel (salt_mi355_nvfp4_matvec_t_dev).  Returns (status, ys[B, R]);
    ys stays 0xFF-filled for a rejected job."""
    lib = init()
    xs = np.ascontiguousarray(xs, np.float32).reshape(-1, C_)
    B = xs.shape[0]
    dw, ds, dx = DeviceBuffer.from_host(packed), DeviceBuffer.from_host(scales), DeviceBuffer.from_host(xs)
    dy, st = DeviceBuffer(B * R * 4, fill=0xFF), DeviceBuffer(4, fill=0)
    stream = lib.salt_mi355_stream()
    check(lib.salt_mi355_nvfp4_matvec_t_dev(dw.ptr, ds.ptr, divisor, input_global_scale, R, C_, B, dx.ptr, dy.ptr, st.ptr,
                                            stream), "nvfp4_matvec_t_dev")
    check(lib.salt_mi355_stream_sync(stream), "sync")
    return int(st.to_host(np.int32)[0]), dy.to_host(np.float32).reshape(B, R)


def nvfp4_matvec_one_launch(packed: np.ndarray, scales: np.ndarray, divisor: float, R: int, C_: int, x: np.ndarray,
                            input_global_scale: float = 64.0, chains: int = 0):
    """The reference matvec of one token with the activation pass inside the
    rows' launch.  Returns (status, y[R]); y stays 0xFF-filled when rejected."""
    lib = init()
    x = np.ascontiguousarray(x, np.float32).reshape(C_)
    dw, ds, dx = DeviceBuffer.from_host(packed), DeviceBuffer.from_host(scales), DeviceBuffer.from_host(x)
    dy, st = DeviceBuffer(R * 4, fill=0xFF), DeviceBuffer(4, fill=0)
    stream = lib.salt_mi355_stream()
    check(lib.salt_mi355_nvfp4_matvec_qdq_dev(dw.ptr, ds.ptr, divisor, input_global_scale, R, C_, dx.ptr, dy.ptr, st.ptr,
                                              chains, stream), "nvfp4_matvec_qdq_dev")
    check(lib.salt_mi355_stream_sync(stream), "sync")
    return int(st.to_host(np.int32)[0]), dy.to_host(np.float32)


def bf16_matvec(weights: np.ndarray, R: int, C_: int, xs: np.ndarray, bias: np.ndarray | None = None,
                weight_offset: int = 0) -> np.ndarray:
    """weights: uint16 [R*C]; xs: float32 [B, C]; returns float32 [B, R].  weight_offset shifts the matrix by that
    many bytes inside its device allocation (the kernels' alignment cases)."""
    lib = init()
    xs = np.ascontiguousarray(xs, np.float32).reshape(-1, C_)
    B = xs.shape[0]
    dw = DeviceBuffer(weights.nbytes + weight_offset + 16, fill=0)
    dw.upload(weights, weight_offset)
    dx, dy = DeviceBuffer.from_host(xs), DeviceBuffer(B * R * 4, fill=0xFF)
    db = DeviceBuffer.from_host(np.ascontiguousarray(bias, np.float32)) if bias is not None else None
    stream = lib.salt_mi355_stream()
    check(lib.salt_mi355_bf16_matvec_dev(dw.at(weight_offset), R, C_, B, dx.ptr, db.ptr if db else None, dy.ptr, stream),
          "bf16_matvec_dev")
    check(lib.salt_mi355_stream_sync(stream), "sync")
    return dy.to_host(np.float32).reshape(B, R)


def q8_matvec(vals: np.ndarray, scales: np.ndarray, biases: np.ndarray | None, R: int, C_: int, xs: np.ndarray,
              value_offset: int = 0) -> np.ndarray:
    """vals: uint8 [R*C]; scales / biases: uint16 per 64 flat elements; xs: float32 [B, C]; returns [B, R]."""
    lib = init()
    xs = np.ascontiguousarray(xs, np.float32).reshape(-1, C_)
    B = xs.shape[0]
    dv = DeviceBuffer(vals.nbytes + value_offset + 16, fill=0)
    dv.upload(vals, value_offset)
    ds = DeviceBuffer.from_host(scales)
    dbi = DeviceBuffer.from_host(biases) if biases is not None else None
    dx, dy = DeviceBuffer.from_host(xs), DeviceBuffer(B * R * 4, fill=0xFF)
    stream = lib.salt_mi355_stream()
    check(lib.salt_mi355_q8_matvec_dev(dv.at(value_offset), ds.ptr, dbi.ptr if dbi else None, R, C_, B, dx.ptr, dy.ptr,
                                       stream), "q8_matvec_dev")
    check(lib.salt_mi355_stream_sync(stream), "sync")
    return dy.to_host(np.float32).reshape(B, R)


def router_topk(logits: np.ndarray, scale: np.ndarray, topk: int, sorted_by_id: bool = False):
    lib = init()
    E = logits.shape[0]
    dl, dsc = DeviceBuffer.from_host(logits.astype(np.float32)), DeviceBuffer.from_host(scale.astype(np.float32))
    sel, w, st = DeviceBuffer(topk * 4, fill=0xEE), DeviceBuffer(topk * 4, fill=0xEE), DeviceBuffer(4, fill=0x7F)
    stream = lib.salt_mi355_stream()
    check(lib.salt_mi355_router_topk_dev(dl.ptr, dsc.ptr, E, topk, int(sorted_by_id), sel.ptr, w.ptr, st.ptr, stream),
          "router_topk_dev")
    check(lib.salt_mi355_stream_sync(stream), "sync")
    return int(st.to_host(np.int32)[0]), sel.to_host(np.int32), w.to_host(np.float32)


def run_cells(cells: list[tuple], arrays: dict[str, np.ndarray]) -> tuple[int, dict[str, np.ndarray]]:
    """Runs a sequence of cells over host arrays.  Each cell is (kind, [names of its views], n, aux, eps, scalar); a
    name maps to one device buffer for the whole sequence (so aliasing is expressed by repeating a name).  Returns the
    status word and every array as it is on the device afterwards."""
    lib = init()
    bufs = {k: DeviceBuffer.from_host(v) for k, v in arrays.items()}
    status = DeviceBuffer(8, fill=0)
    table = (Cell * len(cells))()
    for c, (kind, names, n, aux, eps, scalar) in enumerate(cells):
        views = (vp * 8)(*[bufs[name].ptr if name is not None else None for name in names] + [None] * (8 - len(names)))
        table[c] = Cell(kind, views, n, aux, eps, scalar)
    stream = lib.salt_mi355_stream()
    check(lib.salt_mi355_cells_dev(table, len(cells), status.ptr, stream), "cells_dev")
    check(lib.salt_mi355_stream_sync(stream), "sync")
    return int(status.to_host(np.int32)[0]), {k: b.to_host(arrays[k].dtype) for k, b in bufs.items()}


class FfnBlock:
    """The weights of one layer's feed-forward block (a synth.ffn_layer dictionary) resident in HBM."""

    def __init__(self, w: dict):
        self.lib = init()
        self.H, self.K = w["hidden"], w["topk"]
        self.bufs = {}
        up = lambda name, a: self.bufs.setdefault(name, DeviceBuffer.from_host(a)).ptr
        d = FfnLayerDesc(w["hidden"], w["dense"], w["routed"], w["n_experts"], w["topk"], float(w["eps"]),
                         float(w["layer_scalar"]))
        for name in ("pre_norm", "pre_norm_2", "router_scale", "per_expert_scale", "post_norm_1", "post_norm_2",
                     "post_norm", "pool"):
            setattr(d, name, up(name, w[name]))
        for name in ("dense_gate", "dense_up", "dense_down", "router"):
            setattr(d, name, (vp * 3)(*[up(f"{name}{k}", a) for k, a in enumerate(w[name])]))
        d.expert_stride = w["pool"].nbytes // w["n_experts"]
        self.desc = d
        self.ws = DeviceBuffer(self.lib.salt_mi355_ffn_block_workspace_bytes(C.byref(d)), fill=0)
        self.residual, self.out = DeviceBuffer(self.H * 4), DeviceBuffer(self.H * 4, fill=0xFF)
        self.sel, self.w, self.status = DeviceBuffer(self.K * 4), DeviceBuffer(self.K * 4), DeviceBuffer(4, fill=0x55)

    def enqueue(self, stream):
        return self.lib.salt_mi355_ffn_block_dev(C.byref(self.desc), self.residual.ptr, self.out.ptr, self.sel.ptr,
                                                 self.w.ptr, self.status.ptr, self.ws.ptr, stream)

    def step(self, residual: np.ndarray):
        self.residual.upload(np.ascontiguousarray(residual, np.float32))
        stream = self.lib.salt_mi355_stream()
        check(self.enqueue(stream), "ffn_block_dev")
        check(self.lib.salt_mi355_stream_sync(stream), "sync")
        return (int(self.status.to_host(np.int32)[0]), self.sel.to_host(np.int32), self.w.to_host(np.float32),
                self.out.to_host(np.float32))


class MoeLayer:
    """One layer's expert pool resident in HBM plus the step workspace."""

    def __init__(self, pool: np.ndarray, n_experts: int, hidden: int, routed: int, topk: int, header_bytes: int = 0):
        """header_bytes: bytes in front of expert 0 inside the device allocation (the engine's pool file has 24)."""
        self.lib = init()
        self.E, self.H, self.F, self.K = n_experts, hidden, routed, topk
        self.stride = pool.nbytes // n_experts
        self.header = header_bytes
        self.pool = DeviceBuffer(pool.nbytes + header_bytes, fill=0)
        self.pool.upload(pool, header_bytes)
        self.ws = DeviceBuffer(self.lib.salt_mi355_moe_workspace_bytes(hidden, routed, n_experts, topk), fill=0)
        self.logits, self.scale = DeviceBuffer(n_experts * 4), DeviceBuffer(n_experts * 4)
        self.x, self.out = DeviceBuffer(hidden * 4), DeviceBuffer(hidden * 4)
        self.sel, self.w = DeviceBuffer(topk * 4), DeviceBuffer(topk * 4)
        self.eo = DeviceBuffer(topk * hidden * 4)
        self.tolerance_class = False    # True: salt_mi355_moe_decode_step_t_dev

    def enqueue(self, stream):
        fn = self.lib.salt_mi355_moe_decode_step_t_dev if self.tolerance_class else self.lib.salt_mi355_moe_decode_step_dev
        return fn(
            self.pool.at(self.header), self.stride, self.H, self.F, self.E, self.K, self.logits.ptr, self.scale.ptr, self.x.ptr,
            self.sel.ptr, self.w.ptr, self.eo.ptr, self.out.ptr, self.ws.ptr, stream)

    def step(self, logits, scale, x):
        self.logits.upload(logits.astype(np.float32)); self.scale.upload(scale.astype(np.float32))
        self.x.upload(x.astype(np.float32))
        stream = self.lib.salt_mi355_stream()
        check(self.enqueue(stream), "moe_decode_step_dev")
        check(self.lib.salt_mi355_stream_sync(stream), "sync")
        status = int(self.ws.to_host(np.int32, 1)[0])
        return (status, self.sel.to_host(np.int32), self.w.to_host(np.float32),
                self.eo.to_host(np.float32).reshape(self.K, self.H), self.out.to_host(np.float32))


def q4_matmul(vals, scales, biases, R: int, C_: int, xs: np.ndarray) -> np.ndarray:
    """Host-array convenience around salt_mi355_q4_matmul_dev (MFMA, tolerance class)."""
    lib = init()
    xs = np.ascontiguousarray(xs, np.float32).reshape(-1, C_)
    B = xs.shape[0]
    dv, ds = DeviceBuffer.from_host(vals), DeviceBuffer.from_host(scales)
    db = DeviceBuffer.from_host(biases) if biases is not None else None
    dx, dy = DeviceBuffer.from_host(xs), DeviceBuffer(B * R * 4, fill=0xFF)
    ws = DeviceBuffer(lib.salt_mi355_q4_matmul_workspace_bytes(C_, B))
    stream = lib.salt_mi355_stream()
    check(lib.salt_mi355_q4_matmul_dev(dv.ptr, ds.ptr, db.ptr if db else None, R, C_, B, dx.ptr, dy.ptr, ws.ptr, stream),
          "q4_matmul_dev")
    check(lib.salt_mi355_stream_sync(stream), "sync")
    return dy.to_host(np.float32).reshape(B, R)


class MoePrefill:
    """One MoE layer's experts in HBM plus the workspace of the grouped prefill
    path (salt_mi355_moe_prefill_dev) for up to `tokens` tokens."""

    def __init__(self, pool: np.ndarray, n_experts: int, hidden: int, routed: int, topk: int, tokens: int):
        self.lib = init()
        self.E, self.H, self.F, self.K, self.T = n_experts, hidden, routed, topk, tokens
        self.stride = pool.nbytes // n_experts
        self.pool = DeviceBuffer.from_host(pool)
        self.ws = DeviceBuffer(self.lib.salt_mi355_moe_prefill_workspace_bytes(hidden, routed, n_experts, topk, tokens))
        self.sel, self.w = DeviceBuffer(tokens * topk * 4), DeviceBuffer(tokens * topk * 4)
        self.x, self.out = DeviceBuffer(tokens * hidden * 4), DeviceBuffer(tokens * hidden * 4)
        self.group_rows, self.row_pairs = DeviceBuffer(n_experts * 4), DeviceBuffer(tokens * topk * 4)
        self.status = DeviceBuffer(4)

    def enqueue(self, stream, tokens: int | None = None):
        T = self.T if tokens is None else tokens
        return self.lib.salt_mi355_moe_prefill_dev(self.pool.ptr, self.stride, self.H, self.F, self.E, self.K, T,
                                                   self.sel.ptr, self.w.ptr, self.x.ptr, self.out.ptr,
                                                   self.group_rows.ptr, self.row_pairs.ptr, self.status.ptr,
                                                   self.ws.ptr, stream)

    def run(self, selected: np.ndarray, weights: np.ndarray, xs: np.ndarray):
        """-> (status, outputs [T][hidden], rows per expert, pair index of each grouped row)"""
        T = selected.shape[0]
        assert T <= self.T
        self.sel.upload(np.ascontiguousarray(selected, np.int32))
        self.w.upload(np.ascontiguousarray(weights, np.float32))
        self.x.upload(np.ascontiguousarray(xs, np.float32))
        self.lib.salt_mi355_dev_fill(self.out.ptr, 0xFF, T * self.H * 4)
        stream = self.lib.salt_mi355_stream()
        check(self.enqueue(stream, T), "moe_prefill_dev")
        check(self.lib.salt_mi355_stream_sync(stream), "sync")
        return (int(self.status.to_host(np.int32)[0]), self.out.to_host(np.float32, T * self.H).reshape(T, self.H),
                self.group_rows.to_host(np.int32), self.row_pairs.to_host(np.int32, T * self.K))


def nvfp4_matmul(packed: np.ndarray, scales: np.ndarray, divisor: float, input_global_scale: float, R: int, C_: int,
                 xs: np.ndarray):
    """Host-array convenience around salt_mi355_nvfp4_matmul_dev (MFMA, tolerance class) -> (status, ys [B][R])."""
    lib = init()
    xs = np.ascontiguousarray(xs, np.float32).reshape(-1, C_)
    B = xs.shape[0]
    dp, ds = DeviceBuffer.from_host(packed), DeviceBuffer.from_host(scales)
    dx, dy = DeviceBuffer.from_host(xs), DeviceBuffer(B * R * 4, fill=0xFF)
    ws = DeviceBuffer(lib.salt_mi355_nvfp4_matmul_workspace_bytes(R, C_, B))
    status = DeviceBuffer(4, fill=0x7F)
    stream = lib.salt_mi355_stream()
    check(lib.salt_mi355_nvfp4_matmul_dev(dp.ptr, ds.ptr, divisor, input_global_scale, R, C_, B, dx.ptr, dy.ptr,
                                          status.ptr, ws.ptr, stream), "nvfp4_matmul_dev")
    check(lib.salt_mi355_stream_sync(stream), "sync")
    return int(status.to_host(np.int32)[0]), dy.to_host(np.float32).reshape(B, R)
