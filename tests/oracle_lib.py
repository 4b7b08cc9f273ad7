"""ctypes bindings of the CPU checker (oracle/liboracle.so) and, when it has
been built, of the reference's own C sources for the path
(oracle/_ref/libsaltref.so).  Test-side only."""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
ORACLE_DIR = ROOT / "oracle"

c_f32p = C.POINTER(C.c_float)
c_i32p = C.POINTER(C.c_int)
c_u8p = C.POINTER(C.c_uint8)
vp = C.c_void_p


def ptr(a: np.ndarray | None):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(vp)


class ExpertGeometry(C.Structure):
    _fields_ = [("hidden", C.c_int), ("routed", C.c_int)]


class FfnLayer(C.Structure):
    """Mirror of OrcFfnLayer; keep() holds the arrays its pointers name."""
    _fields_ = [("hidden", C.c_int), ("dense", C.c_int), ("routed", C.c_int), ("n_experts", C.c_int), ("topk", C.c_int),
                ("eps", C.c_float), ("layer_scalar", C.c_float),
                ("pre_norm", vp), ("pre_norm_2", vp), ("router_scale", vp), ("per_expert_scale", vp),
                ("post_norm_1", vp), ("post_norm_2", vp), ("post_norm", vp),
                ("dense_gate", vp * 3), ("dense_up", vp * 3), ("dense_down", vp * 3), ("router", vp * 3), ("pool", vp)]


def ffn_layer_struct(w: dict) -> FfnLayer:
    """OrcFfnLayer over the arrays of a synth.ffn_layer() dictionary (which must outlive it)."""
    at = lambda a: a.ctypes.data
    L = FfnLayer(w["hidden"], w["dense"], w["routed"], w["n_experts"], w["topk"], float(w["eps"]), float(w["layer_scalar"]))
    for name in ("pre_norm", "pre_norm_2", "router_scale", "per_expert_scale", "post_norm_1", "post_norm_2", "post_norm",
                 "pool"):
        setattr(L, name, at(w[name]))
    for name in ("dense_gate", "dense_up", "dense_down", "router"):
        setattr(L, name, (vp * 3)(*[at(a) for a in w[name]]))
    return L


def _sig(fn, restype, *argtypes):
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


def load_oracle() -> C.CDLL:
    so = ORACLE_DIR / "liboracle.so"
    src = ORACLE_DIR / "salt_oracle.c"
    if not so.exists() or so.stat().st_mtime < src.stat().st_mtime:
        subprocess.check_call(["make", "-C", str(ORACLE_DIR), "liboracle.so"],
                              stdout=subprocess.DEVNULL)
    lib = C.CDLL(str(so))
    i, f, d, sz = C.c_int, C.c_float, C.c_double, C.c_size_t
    _sig(lib.orc_bf16, f, C.c_uint16)
    _sig(lib.orc_q4_decode, None, vp, vp, vp, sz, vp)
    _sig(lib.orc_q4_row, f, vp, vp, vp, i, vp, i)
    _sig(lib.orc_q4_matvec, i, vp, vp, vp, i, i, vp, vp)
    _sig(lib.orc_q4_matvec_rows, i, vp, vp, vp, i, i, vp, vp, i, i)
    _sig(lib.orc_q4_matvec_batch, i, vp, vp, vp, i, i, i, vp, vp)
    _sig(lib.orc_q4_matvec_threads, i, vp, vp, vp, i, i, vp, vp, i)
    _sig(lib.orc_bf16_matvec, None, vp, i, i, vp, vp, vp)
    _sig(lib.orc_q8_matvec, None, vp, vp, vp, i, i, vp, vp)
    _sig(lib.orc_e2m1, f, C.c_uint8)
    _sig(lib.orc_e4m3fn, f, C.c_uint8)
    _sig(lib.orc_e4m3fn_encode, i, f, c_u8p)
    _sig(lib.orc_e2m1_encode, C.c_uint8, f)
    _sig(lib.orc_e4m3fn_encode_rne, C.c_uint8, f)
    _sig(lib.orc_e2m1_encode_rne, C.c_uint8, f)
    _sig(lib.orc_nvfp4_qdq, i, vp, i, f, vp, vp, vp)
    _sig(lib.orc_nvfp4_dequant_weights, i, vp, vp, f, i, i, vp)
    _sig(lib.orc_nvfp4_row, f, vp, vp, f, i, i, vp)
    _sig(lib.orc_nvfp4_matvec, i, vp, vp, f, f, i, i, vp, vp, vp, vp, vp)
    _sig(lib.orc_nvfp4_matvec_weights_only, i, vp, vp, f, i, i, vp, vp)
    _sig(lib.orc_expf, f, f)
    _sig(lib.orc_tanhf, f, f)
    _sig(lib.orc_gelu_tanh, f, f)
    _sig(lib.orc_router_topk, i, vp, vp, i, i, vp, vp)
    _sig(lib.orc_sort_selection, None, vp, vp, i)
    _sig(lib.orc_mix64, C.c_uint64, C.c_uint64)
    _sig(lib.orc_router_fixture, i, vp, vp, i, i, C.c_uint64, i, d)
    _sig(lib.orc_rsqrtf, f, f)
    _sig(lib.orc_sqrtf, f, f)
    _sig(lib.orc_pow_minus_half, f, f)
    _sig(lib.orc_rmsnorm, i, vp, vp, vp, i, f, i)
    _sig(lib.orc_router_input, i, vp, vp, vp, i, f)
    _sig(lib.orc_residual_postnorm, i, vp, vp, vp, vp, i, f)
    _sig(lib.orc_parallel_ffn_combine, i, vp, vp, vp, vp, vp, vp, vp, f, i, f)
    _sig(lib.orc_softcap, i, vp, i, f)
    _sig(lib.orc_ffn_block, i, C.POINTER(FfnLayer), vp, vp, vp, vp, i)
    G = C.POINTER(ExpertGeometry)
    _sig(lib.orc_expert_proj_bytes, sz, G)
    _sig(lib.orc_expert_slot_bytes, sz, G)
    _sig(lib.orc_expert_ffn, i, G, vp, vp, vp, vp, vp)
    _sig(lib.orc_moe_decode_step, i, G, vp, i, i, vp, vp, vp, vp, vp, vp, vp, i)
    _sig(lib.orc_moe_group, i, G, vp, i, i, i, vp, vp, vp, vp, vp, i)
    return lib


def load_reference() -> C.CDLL | None:
    """The reference's own sources compiled by `make -C oracle ref`; None when
    that library has not been built (the tests that need it skip)."""
    so = ORACLE_DIR / "_ref" / "libsaltref.so"
    if not so.exists():
        return None
    lib = C.CDLL(str(so))
    i, f, d = C.c_int, C.c_float, C.c_double
    _sig(lib.salt_q4_decode, None, vp, vp, vp, i, vp)
    _sig(lib.salt_q4_matvec, None, vp, vp, vp, i, i, vp, vp)
    _sig(lib.salt_q4_matvec_status, i, vp, vp, vp, i, i, vp, vp)
    _sig(lib.salt_q4_matvec_rows_status, i, vp, vp, vp, i, i, vp, vp, i, i)
    _sig(lib.salt_q4_matvec_batch_rows, i, vp, vp, vp, i, i, i, vp, vp, i, i)
    _sig(lib.salt_bf16_matvec, None, vp, i, i, vp, vp, vp)
    _sig(lib.salt_q8_matvec, None, vp, vp, vp, i, i, vp, vp)
    _sig(lib.salt_kernels_set_simd, None, i)
    _sig(lib.salt_kernels_set_in_expert, None, i)
    _sig(lib.salt_nvfp4_e2m1, f, C.c_uint8)
    _sig(lib.salt_nvfp4_e4m3fn, f, C.c_uint8)
    _sig(lib.salt_nvfp4_e4m3fn_encode, i, f, c_u8p)
    _sig(lib.salt_nvfp4_quantize_input_reference, i, vp, i, f, vp, vp, vp)
    _sig(lib.salt_nvfp4_dequantize_weights_reference, i, vp, vp, f, i, i, vp)
    _sig(lib.salt_nvfp4_matvec_reference, i, vp, vp, f, f, i, i, vp, vp, vp, vp, vp)
    _sig(lib.salt_expf, f, f)
    _sig(lib.salt_tanhf, f, f)
    _sig(lib.salt_gemma4_gelu_tanh, f, f)
    _sig(lib.salt_gemma4_router_topk, i, vp, vp, i, i, vp, vp)
    _sig(lib.salt_mix64, C.c_uint64, C.c_uint64)
    _sig(lib.salt_rsqrtf, f, f)
    _sig(lib.salt_sqrtf, f, f)
    _sig(lib.salt_powf, f, f, f)
    _sig(lib.salt_gemma4_rmsnorm, i, vp, vp, vp, i, f, i)
    _sig(lib.salt_gemma4_router_input, i, vp, vp, vp, i, f)
    _sig(lib.salt_gemma4_residual_postnorm, i, vp, vp, vp, vp, i, f)
    _sig(lib.salt_gemma4_parallel_ffn_combine, i, vp, vp, vp, vp, vp, vp, vp, f, i, f, vp)
    _sig(lib.salt_gemma4_softcap, i, vp, i, f)
    if hasattr(lib, "refdrv_moe_decode_step"):          # oracle/ref_moe_driver.c, compiled into the same library
        _sig(lib.refdrv_moe_decode_step, i, vp, C.c_size_t, i, i, i, i, vp, vp, vp, vp, vp, vp, vp, vp, i)
        _sig(lib.refdrv_moe_group, i, vp, C.c_size_t, i, i, i, i, i, vp, vp, vp, vp, vp)
    return lib


def bits(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def host_threads() -> int:
    return max(1, min(16, len(os.sched_getaffinity(0))))
