#!/usr/bin/env python3
"""Writes tests/golden/*.npz from the reference's own C sources.

Run in a container that has the reference tree mounted:

    make -C oracle ref && python tests/golden/make_golden.py

The reference sources are compiled where they lie into
oracle/_ref/libsaltref.so (see oracle/Makefile) and called through ctypes; this
script holds no reference code, only calls of its public functions.  Inputs are
regenerated from seeds by the package's own generator (salt-core_amd/synth.py);
each fixture stores a digest of its input bytes so that generator drift is
noticed, and the reference's outputs as raw bit patterns.
"""
from __future__ import annotations

import ctypes as C
import hashlib
import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
sys.path[:0] = [str(ROOT), str(ROOT / "tests")]

from __graft_entry__ import load_package  # noqa: E402
from oracle_lib import bits, load_reference, ptr, vp  # noqa: E402

synth = load_package().synth
from golden.cases import (GROUP_CASES, MOE_CASES, NVFP4_MATVEC_CASES, NVFP4_QDQ_CASES, Q4_CASES,  # noqa: E402
                          digest, nvfp4_qdq_input, pool_digest, q4_case_inputs)
ref = load_reference()
if ref is None:
    sys.exit("oracle/_ref/libsaltref.so missing: run `make -C oracle ref` first")


# ---------------------------------------------------------------- Q4 matvec
def make_q4():
    out = {}
    for name, R, C, B, wseed, xseed, stride in Q4_CASES:
        vals, scales, biases, xs = q4_case_inputs(R, C, B, wseed, xseed)
        ys = np.zeros((B, R), np.float32)
        # per-token salt_q4_matvec_status, default threads (the batch entry
        # points reduce to exactly this on x86, src/kernels.c:1252-1261)
        for t in range(B):
            assert ref.salt_q4_matvec_status(ptr(vals), ptr(scales), ptr(biases), R, C,
                                             ptr(xs[t]), ptr(ys[t])) == 0
        rows = np.arange(0, R, stride, dtype=np.int32)
        out[name + ".rows"] = rows
        out[name + ".y_bits"] = bits(ys)[:, rows]
        out[name + ".digest"] = np.array(digest(vals, scales, biases, xs))
    np.savez_compressed(HERE / "q4_matvec.npz", **out)


# ---------------------------------------------------------------- bitmath
def make_math():
    g = synth.rng(2024)
    x = np.concatenate([
        g.uniform(-90, 90, 1500), g.uniform(-12, 12, 1500), g.standard_normal(1500),
        g.standard_normal(500) * 1e-3,
        [0.0, -0.0, 88.722839, 88.72284, -87.336548, -87.33655, 10.0, -10.0, 9.999999, -9.999999,
         0.34657359, -0.34657359, 0.6931472, 1.0, -1.0, 1e-30, -1e-30]]).astype(np.float32)
    e = np.array([ref.salt_expf(float(v)) for v in x], np.float32)
    t = np.array([ref.salt_tanhf(float(v)) for v in x], np.float32)
    ge = np.array([ref.salt_gemma4_gelu_tanh(float(v)) for v in x], np.float32)
    np.savez_compressed(HERE / "bitmath.npz", x_bits=bits(x), expf_bits=bits(e), tanhf_bits=bits(t),
                        gelu_bits=bits(ge))


# ---------------------------------------------------------------- routers
class SaltCfg(C.Structure):     # field list of include/salt/salt.h:56-79
    _fields_ = [(n, C.c_int) for n in (
        "n_layers", "n_experts", "topk", "n_shared", "hidden", "latent", "moe_inter", "n_heads",
        "n_kv_heads", "qk_rope", "linear_num_key_heads", "linear_num_value_heads",
        "linear_key_head_dim", "linear_value_head_dim")] + [
        (n, C.c_double) for n in ("rope_factor", "rope_beta_fast", "rope_beta_slow", "rope_max_pos",
                                  "rope_theta")] + [
        ("expert_nbytes", C.c_int64), ("n_shards", C.c_int), ("seed", C.c_uint64)]


def make_router():
    N, E, K = 24, 128, 8
    g = synth.rng(77)
    logits = g.standard_normal((N, E)).astype(np.float32)
    logits[1::3] = (np.round(logits[1::3] * 2) / 2).astype(np.float32)     # ties
    logits[2] = 0.0                                                        # all equal
    scale = g.uniform(0.25, 4.0, (N, E)).astype(np.float32)
    scale[::2] = 1.0
    sel = np.zeros((N, K), np.int32); w = np.zeros((N, K), np.float32)
    for i in range(N):
        assert ref.salt_gemma4_router_topk(ptr(logits[i]), ptr(scale[i]), E, K, ptr(sel[i]), ptr(w[i])) == 0
    out = dict(logits_bits=bits(logits), scale_bits=bits(scale), selected=sel, weight_bits=bits(w))
    # fixture router (src/router.c)
    ref.salt_router.restype = None
    ref.salt_router.argtypes = [vp, vp, C.POINTER(SaltCfg), C.c_uint64, C.c_int, C.c_double]
    cfg = SaltCfg(); cfg.n_experts = 128; cfg.topk = 8
    states = np.array([0, 1, 0x1234567890ABCDEF, 2 ** 64 - 1, 42, 0xB1A5], np.uint64)
    layers = np.array([0, 3, 17, 29, 5, 11], np.int32)
    local = np.array([0.0, 0.0, 0.75, 0.0, 2.0, 0.1])
    fidx = np.zeros((len(states), 8), np.int32); fw = np.zeros((len(states), 8), np.float32)
    for i in range(len(states)):
        ref.salt_router(ptr(fidx[i]), ptr(fw[i]), C.byref(cfg), int(states[i]), int(layers[i]), float(local[i]))
    out.update(fx_states=states, fx_layers=layers, fx_locality=local, fx_idx=fidx, fx_w_bits=bits(fw))
    np.savez_compressed(HERE / "router.npz", **out)


# ---------------------------------------------------------------- NVFP4
def make_nvfp4():
    out = {}
    g = synth.rng(88)
    v = np.concatenate([g.uniform(-460, 460, 3000), g.standard_normal(3000) * 0.01,
                        g.standard_normal(1000) * 1e-3, [0.0, -0.0, 448.0, 449.0, 1e9, -1e9,
                                                         0.0009765625, 0.0029296875, 0.015625, 0.0146484375]]
                       ).astype(np.float32)
    codes = np.zeros(len(v), np.uint8)
    c = C.c_uint8(0)
    for i, x in enumerate(v):
        assert ref.salt_nvfp4_e4m3fn_encode(float(x), C.byref(c)) == 0
        codes[i] = c.value
    out["enc_x_bits"] = bits(v); out["enc_codes"] = codes
    for tag, gscale, seed in NVFP4_QDQ_CASES:
        x = nvfp4_qdq_input(tag, seed)
        p = np.zeros(4096, np.uint8); s = np.zeros(512, np.uint8); d = np.zeros(8192, np.float32)
        assert ref.salt_nvfp4_quantize_input_reference(ptr(x), 8192, gscale, ptr(p), ptr(s), ptr(d)) == 0
        out[f"qdq_{tag}.packed"] = p; out[f"qdq_{tag}.scales"] = s; out[f"qdq_{tag}.dequant_bits"] = bits(d)
        out[f"qdq_{tag}.digest"] = np.array(digest(x))
    for name, R, Cc, wseed, xseed, divisor, gscale in NVFP4_MATVEC_CASES:
        packed, scales = synth.nvfp4_tensor(R, Cc, wseed)
        x = synth.activations(Cc, 1, xseed)[0]
        y = np.zeros(R, np.float32)
        xp = np.zeros(Cc // 2, np.uint8); xs = np.zeros(Cc // 16, np.uint8); xd = np.zeros(Cc, np.float32)
        assert ref.salt_nvfp4_matvec_reference(ptr(packed), ptr(scales), divisor, gscale, R, Cc, ptr(x), ptr(y),
                                               ptr(xp), ptr(xs), ptr(xd)) == 0
        out[name + ".y_bits"] = bits(y)
        out[name + ".digest"] = np.array(digest(packed, scales, x))
    np.savez_compressed(HERE / "nvfp4.npz", **out)


# ---------------------------------------------------------------- MoE decode step
def ref_expert(pool, expert, H, F, x):
    """gate, up, gelu*up, down through the reference's public functions in the
    order of its expert worker (gemma4_text.c:7608-7649)."""
    gate = np.zeros(F, np.float32); up = np.zeros(F, np.float32); out = np.zeros(H, np.float32)
    gv = synth.expert_views(pool, expert, 0, H, F)
    uv = synth.expert_views(pool, expert, 1, H, F)
    dv = synth.expert_views(pool, expert, 2, H, F)
    ref.salt_kernels_set_in_expert(1)
    ref.salt_q4_matvec(ptr(gv[0]), ptr(gv[1]), ptr(gv[2]), F, H, ptr(x), ptr(gate))
    ref.salt_q4_matvec(ptr(uv[0]), ptr(uv[1]), ptr(uv[2]), F, H, ptr(x), ptr(up))
    for i in range(F):
        gate[i] = np.float32(ref.salt_gemma4_gelu_tanh(float(gate[i]))) * up[i]
    ref.salt_q4_matvec(ptr(dv[0]), ptr(dv[1]), ptr(dv[2]), H, F, ptr(gate), ptr(out))
    ref.salt_kernels_set_in_expert(0)
    return gate, out


def sort_pairs(sel, w):
    order = np.argsort(sel, kind="stable")
    return sel[order].copy(), w[order].copy()


def make_moe():
    out = {}
    for name, E, K, H, F, pseed, lseed, xseed in MOE_CASES:
        pool = synth.expert_pool(E, H, F, pseed)
        logits = synth.router_logits(E, lseed)
        scale = np.ones(E, np.float32)
        x = synth.activations(H, 1, xseed)[0]
        sel = np.zeros(K, np.int32); w = np.zeros(K, np.float32)
        assert ref.salt_gemma4_router_topk(ptr(logits), ptr(scale), E, K, ptr(sel), ptr(w)) == 0
        sel, w = sort_pairs(sel, w)
        eo = np.zeros((K, H), np.float32); acts = np.zeros((K, F), np.float32)
        for i in range(K):
            acts[i], eo[i] = ref_expert(pool, int(sel[i]), H, F, x)
        y = np.zeros(H, np.float32)
        for i in range(K):                       # gemma4_text.c:8301-8304
            y = (y + (eo[i] * w[i]).astype(np.float32)).astype(np.float32)
        out[name + ".selected"] = sel; out[name + ".weight_bits"] = bits(w)
        out[name + ".act_bits"] = bits(acts); out[name + ".expert_out_bits"] = bits(eo)
        out[name + ".y_bits"] = bits(y)
        out[name + ".digest"] = np.array(pool_digest(pool, logits, x))
    np.savez_compressed(HERE / "moe_decode.npz", **out)


# ---------------------------------------------------------------- grouped MoE
class Scratch(C.Structure):     # include/salt/moe_group.h:8-24
    _fields_ = [("used", vp), ("acquired", vp), ("leases", vp), ("batch_leases", vp), ("run_leases", vp),
                ("expert_ids", vp), ("run_groups", vp), ("group_inputs", vp), ("group_outputs", vp),
                ("selection_outputs", vp), ("expert_capacity", C.c_size_t), ("acquire_capacity", C.c_size_t),
                ("run_capacity", C.c_size_t), ("group_element_capacity", C.c_size_t),
                ("selection_element_capacity", C.c_size_t)]


class Job(C.Structure):         # include/salt/moe_group.h:29-39
    _fields_ = [("batch", C.c_int), ("topk", C.c_int), ("n_experts", C.c_int), ("hidden", C.c_int),
                ("selected", vp), ("weights", vp), ("inputs", vp), ("outputs", vp),
                ("scratch", C.POINTER(Scratch))]


ACQ = C.CFUNCTYPE(C.c_int, vp, C.c_int, C.POINTER(vp))
ACQM = C.CFUNCTYPE(C.c_int, vp, C.POINTER(C.c_int), C.c_int, C.POINTER(vp))
RUN = C.CFUNCTYPE(C.c_int, vp, C.c_int, vp, C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_float))
RUNM = C.CFUNCTYPE(C.c_int, vp, C.POINTER(C.c_int), C.POINTER(vp), C.POINTER(C.c_int), C.c_int,
                   C.POINTER(C.c_float), C.POINTER(C.c_float))
REL = C.CFUNCTYPE(C.c_int, vp, C.c_int, vp)


class Ops(C.Structure):         # include/salt/moe_group.h:41-59
    _fields_ = [("acquire", ACQ), ("acquire_many", ACQM), ("acquire_batch", C.c_int), ("run", RUN),
                ("run_many", RUNM), ("run_batch", C.c_int), ("release", REL)]


def make_group():
    out = {}
    ref.salt_moe_group_execute.restype = C.c_int
    ref.salt_moe_group_execute.argtypes = [C.POINTER(Job), C.POINTER(Ops), vp]
    for name, T, E, K, H, F, run_batch, pseed, sseed in GROUP_CASES:
        pool = synth.expert_pool(E, H, F, pseed)
        sel, w = synth.zipf_selection(T, E, K, 1.1, sseed)
        xs = synth.activations(H, T, sseed + 1)
        ys = np.zeros((T, H), np.float32)
        order = []            # (expert, rows) in the order the engine ran them

        def run_rows(expert, rows, inp, outp):
            a = np.ctypeslib.as_array(inp, shape=(rows, H))
            b = np.ctypeslib.as_array(outp, shape=(rows, H))
            for r in range(rows):
                _, b[r] = ref_expert(pool, expert, H, F, np.ascontiguousarray(a[r]))

        def acquire(ctx, expert, lease):
            lease[0] = expert + 1
            return 0

        def run(ctx, expert, lease, group, inp, outp):
            order.append((expert, group))
            run_rows(expert, group, inp, outp)
            return 0

        def run_many(ctx, experts, leases, groups, count, inp, outp):
            at = 0
            for i in range(count):
                order.append((experts[i], groups[i]))
                run_rows(experts[i], groups[i],
                         C.cast(C.addressof(inp.contents) + at * H * 4, C.POINTER(C.c_float)),
                         C.cast(C.addressof(outp.contents) + at * H * 4, C.POINTER(C.c_float)))
                at += groups[i]
            return 0

        def release(ctx, expert, lease):
            return 0

        used = np.zeros(E, np.uint8); acq = np.zeros(E, np.uint8)
        leases = np.zeros(E, np.uint64); bl = np.zeros(E, np.uint64); rl = np.zeros(E, np.uint64)
        ids = np.zeros(E, np.int32); rg = np.zeros(E, np.int32)
        gi = np.zeros(T * K * H, np.float32); go = np.zeros(T * K * H, np.float32)
        so = np.zeros(T * K * H, np.float32)
        scratch = Scratch(ptr(used), ptr(acq), ptr(leases), ptr(bl), ptr(rl), ptr(ids), ptr(rg), ptr(gi),
                          ptr(go), ptr(so), E, E, E, T * K * H, T * K * H)
        job = Job(T, K, E, H, ptr(sel), ptr(w), ptr(xs), ptr(ys), C.pointer(scratch))
        ops = Ops(ACQ(acquire), ACQM(), 0, RUN(run) if not run_batch else RUN(),
                  RUNM(run_many) if run_batch else RUNM(), run_batch, REL(release))
        ctx = C.c_int(0)
        assert ref.salt_moe_group_execute(C.byref(job), C.byref(ops), C.cast(C.byref(ctx), vp)) == 0
        out[name + ".selected"] = sel; out[name + ".weight_bits"] = bits(w)
        out[name + ".y_bits"] = bits(ys)
        out[name + ".run_experts"] = np.array([e for e, _ in order], np.int32)
        out[name + ".run_rows"] = np.array([r for _, r in order], np.int32)
        out[name + ".digest"] = np.array(pool_digest(pool, xs))
    np.savez_compressed(HERE / "moe_group.npz", **out)


if __name__ == "__main__":
    which = sys.argv[1:] or ["q4", "math", "router", "nvfp4", "moe", "group"]
    table = dict(q4=make_q4, math=make_math, router=make_router, nvfp4=make_nvfp4, moe=make_moe,
                 group=make_group)
    for key in which:
        table[key]()
        print("wrote", key, flush=True)
