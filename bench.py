#!/usr/bin/env python3
"""Throughput of the affine-Q4 decode matvec path on one MI355X.

A step is one pass of the decode-shape sweep (BASELINE.json configs[1], batch
1): for each (K, N) in {(2816, 2816), (2816, 16384), (8192, 2816)} one launch
of the tolerance-class Q4 kernel (per-group affine form with exact integer dot
products; stated bound in include/salt_gpu_mi355.h) over G distinct weight
instances resident in HBM
(G chosen so that every launch streams more than the 256 MB Infinity Cache can
hold), the way the engine's batched entry point dispatches many matrices at
once (reference salt_gpu_q4_batch, include/salt/gpu.h:83).  `value` is the
algorithmic bytes of a step (0.5625 B per weight element plus activations and
outputs) divided by the step time, weights already resident when the timed
region starts.

The JSON line also carries the roofline of the dominant kernel (achieved HBM
GB/s against 8 TB/s), the same sweep timed on the host cores with the
reference's own C kernel when oracle/_ref is present (else the checker's
port), and, under "extra", the same sweep on the bit-exact kernel, the MoE
decode layer-step, the NVFP4 matvec and the batch-4 sweeps.

--only NAME runs a single leg (sweep, sweep-exact, sweep-b4, single, single-exact, moe, moe-t, prefill, ffn, abi, nvfp4-t, nvfp4-b256, copy): what the
rocprofv3 commands in profiles/ use.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path[:0] = [str(ROOT), str(ROOT / "tests")]

MFMA_BF16_PEAK_TFLOPS = 2500.0
HBM_PEAK_GBS = 8000.0
SWEEP = [(2816, 2816), (16384, 2816), (2816, 8192)]        # (R, C) = (N, K)
INSTANCE_BYTES = 640e6                                      # distinct weight bytes per launch
# HBM bytes one launch of the sweep moves (mean of the three launches), from FETCH_SIZE / WRITE_SIZE counter runs scaled
# by a copy of known size; taken from the profile summary named beside it, for the default instance counts only, keyed
# by kernel family and tokens per activation batch.  bench.py does not measure it: it reports it with its source.
TRAFFIC_FROM_PROFILE = {
    ("q4_dot16_kernel", 1): (650_600_000, "profiles/q4_dot16_kernel_decode_sweep.md"),
    ("q4_dot16_kernel", 4): (656_500_000, "profiles/q4_dot16_kernel_decode_sweep.md"),
    ("q4_tile_kernel", 1): (661_200_000, "profiles/q4_tile_kernel_decode_sweep_b1.md"),
}


class Events:
    def __init__(self, lib, stream):
        self.lib, self.stream = lib, stream
        self.a, self.b = lib.salt_mi355_event_create(), lib.salt_mi355_event_create()

    def start(self):
        self.lib.salt_mi355_event_record(self.a, self.stream)

    def stop_ms(self) -> float:
        self.lib.salt_mi355_event_record(self.b, self.stream)
        ms = C.c_float()
        assert self.lib.salt_mi355_event_elapsed_ms(self.a, self.b, C.byref(ms)) == 0
        return float(ms.value)


class Q4Sweep:
    """The three decode shapes, G instances each, one multi-job launch per shape."""

    def __init__(self, gpu, synth, tokens: int, distinct: int = 0, exact: bool = False):
        """distinct > 0: the same number of jobs, but only that many weight instances in memory (cache-warm).
        exact: the bit-exact kernel (salt_mi355_q4_jobs_dev) instead of the tolerance-class one."""
        self.gpu, self.lib, self.tokens, self.exact = gpu, gpu.load(), tokens, exact
        self.launches, self.keep = [], []
        self.bytes_per_step = 0
        for seed, (R, Cc) in enumerate(SWEEP):
            vals, scales, biases = synth.q4_tensor(R, Cc, 100 + seed)
            per = vals.nbytes + scales.nbytes + biases.nbytes
            G = max(2, int(INSTANCE_BYTES // per))
            copies = min(G, distinct) if distinct > 0 else G
            weights = gpu.DeviceBuffer(per * copies)
            for g in range(copies):
                weights.upload(vals, g * per)
                weights.upload(scales, g * per + vals.nbytes)
                weights.upload(biases, g * per + vals.nbytes + scales.nbytes)
            xs = gpu.DeviceBuffer.from_host(synth.activations(Cc, tokens, 200 + seed))
            ys = gpu.DeviceBuffer(G * tokens * R * 4)
            jobs = (gpu.Q4Job * G)()
            for g in range(G):
                at = (g % copies) * per
                jobs[g] = gpu.Q4Job(weights.at(at), weights.at(at + vals.nbytes),
                                    weights.at(at + vals.nbytes + scales.nbytes), xs.ptr,
                                    ys.at(g * tokens * R * 4), R)
            self.keep += [weights, xs, ys]
            self.launches.append((jobs, G, Cc))
            self.bytes_per_step += G * synth.q4_bytes(R, Cc, tokens)

    def single_launches(self, shape: int, stream):
        """Every instance of one shape as a launch of its own (what the engine's salt_gpu_q4_matvec issues)."""
        jobs, G, Cc = self.launches[shape]
        for g in range(G):
            j = jobs[g]
            if self.exact:
                rc = self.lib.salt_mi355_q4_matvec_dev(j.vals, j.scales, j.biases, j.rows, Cc, self.tokens, j.xs, j.ys, 0,
                                                       stream)
            else:
                rc = self.lib.salt_mi355_q4_matvec_t_dev(j.vals, j.scales, j.biases, j.rows, Cc, self.tokens, j.xs, j.ys,
                                                         stream)
            if rc != 0:
                raise RuntimeError(self.lib.salt_mi355_last_error().decode())
        return G

    def step(self, stream):
        for jobs, G, Cc in self.launches:
            if self.exact:
                rc = self.lib.salt_mi355_q4_jobs_dev(jobs, G, Cc, self.tokens, 0, stream)
            else:
                rc = self.lib.salt_mi355_q4_jobs_t_dev(jobs, G, Cc, self.tokens, stream)
            if rc != 0:
                raise RuntimeError(self.lib.salt_mi355_last_error().decode())


def timed(lib, stream, events, fn, warmup, steps):
    for _ in range(warmup):
        fn(stream)
    assert lib.salt_mi355_stream_sync(stream) == 0
    events.start()
    for _ in range(steps):
        fn(stream)
    ms = events.stop_ms()
    assert lib.salt_mi355_stream_sync(stream) == 0
    return ms / steps


def cpu_baseline(synth, budget_s: float = 12.0):
    """The same sweep (one instance per shape, batch 1) on the host cores."""
    from oracle_lib import load_oracle, load_reference, ptr
    cores = max(1, min(16, len(os.sched_getaffinity(0))))
    os.environ.setdefault("SALT_ATTN_THREADS", str(cores))
    ref = load_reference()
    oracle = load_oracle()
    cases = []
    for seed, (R, Cc) in enumerate(SWEEP):
        vals, scales, biases = synth.q4_tensor(R, Cc, 100 + seed)
        x = synth.activations(Cc, 1, 200 + seed)[0]
        cases.append((R, Cc, vals, scales, biases, x, np.zeros(R, np.float32)))

    def one_pass():
        for R, Cc, vals, scales, biases, x, y in cases:
            if ref is not None:
                ref.salt_q4_matvec(ptr(vals), ptr(scales), ptr(biases), R, Cc, ptr(x), ptr(y))
            else:
                oracle.orc_q4_matvec_threads(ptr(vals), ptr(scales), ptr(biases), R, Cc, ptr(x), ptr(y), cores)

    one_pass()
    t0 = time.perf_counter()
    one_pass()
    once = time.perf_counter() - t0
    reps = max(3, min(20000, int(budget_s / max(once, 1e-6))))
    t0 = time.perf_counter()
    for _ in range(reps):
        one_pass()
    elapsed = time.perf_counter() - t0
    nbytes = sum(synth.q4_bytes(R, Cc, 1) for R, Cc in SWEEP)
    threads = int(os.environ["SALT_ATTN_THREADS"]) if ref is not None else cores
    # one thread: the reference's SIMD kernel without its row split (its expert-scope switch), else the scalar port
    if ref is not None:
        ref.salt_kernels_set_in_expert(1)
    t0 = time.perf_counter()
    single_reps = 0
    while time.perf_counter() - t0 < 2.0:
        for R, Cc, vals, scales, biases, x, y in cases:
            if ref is not None:
                ref.salt_q4_matvec(ptr(vals), ptr(scales), ptr(biases), R, Cc, ptr(x), ptr(y))
            else:
                oracle.orc_q4_matvec_threads(ptr(vals), ptr(scales), ptr(biases), R, Cc, ptr(x), ptr(y), 1)
        single_reps += 1
    single = nbytes * single_reps / (time.perf_counter() - t0) / 1e9
    if ref is not None:
        ref.salt_kernels_set_in_expert(0)
    return {
        "single_thread": {"value": round(single, 3), "unit": "GB/s", "cores": 1,
                          "kind": "reference" if ref is not None else "port",
                          "sample": f"{single_reps} passes of the same sweep"},
        "value": round(nbytes * reps / elapsed / 1e9, 3), "unit": "GB/s", "cores": threads,
        "kind": "reference" if ref is not None else "port",
        "sample": f"{reps} passes of the 3-shape sweep, one weight instance per shape, batch 1, "
                  f"{elapsed:.1f} s; the reference row-splits over {threads} threads when R >= 2048",
    }


def cpu_other_configs(synth, pool, cores: int, budget_s: float = 3.0):
    """The other configurations on the host cores, each on a bounded sample."""
    import ctypes as C
    from oracle_lib import ExpertGeometry, load_oracle, load_reference, ptr
    oracle, ref = load_oracle(), load_reference()
    out = {}

    def rate(fn, unit_count, budget):
        fn()
        t0 = time.perf_counter(); fn(); once = time.perf_counter() - t0
        reps = max(1, min(1000, int(budget / max(once, 1e-6))))
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        return unit_count * reps / (time.perf_counter() - t0), reps

    # BASELINE configs[0] (one 4096 x 4096 matvec) and the batch-4 sweep with the reference's own salt_q4_matvec (its
    # x86 batch path decodes the weights once per token, so four tokens are four calls)
    if ref is not None:
        v0, s0, b0 = synth.q4_tensor(4096, 4096, 60)
        x0, y0 = synth.activations(4096, 1, 61)[0], np.zeros(4096, np.float32)
        calls_per_s, reps = rate(lambda: ref.salt_q4_matvec(ptr(v0), ptr(s0), ptr(b0), 4096, 4096, ptr(x0), ptr(y0)), 1,
                                 budget_s)
        out["q4_4096_matvec_us"] = {"value": round(1e6 / calls_per_s, 1), "kind": "reference", "cores": cores,
                                    "sample": f"{reps} calls"}
        sweep_cases = []
        for seed, (R, Cc) in enumerate(SWEEP):
            vals, scales, biases = synth.q4_tensor(R, Cc, 100 + seed)
            sweep_cases.append((R, Cc, vals, scales, biases, synth.activations(Cc, 4, 200 + seed), np.zeros((4, R), np.float32)))

        def batch4_pass():
            for R, Cc, vals, scales, biases, xs4, ys4 in sweep_cases:
                for t in range(4):
                    ref.salt_q4_matvec(ptr(vals), ptr(scales), ptr(biases), R, Cc, ptr(xs4[t]), ptr(ys4[t]))

        nbytes4 = sum(synth.q4_bytes(R, Cc, 4) for R, Cc in SWEEP)
        bytes_per_s, reps = rate(batch4_pass, nbytes4, budget_s)
        out["q4_sweep_batch4_gbps"] = {"value": round(bytes_per_s / 1e9, 3), "kind": "reference", "cores": cores,
                                       "sample": f"{reps} passes of the 3-shape sweep at batch 4 (one call per token)"}
    # MoE decode layer-step and grouped prefill: the reference's own public functions in the order of its (static)
    # step, driven by oracle/ref_moe_driver.c; experts on min(cores, 8) threads as gemma4_text.c:8247-8277
    E, K, H, F = 128, 8, 2816, 704
    g = ExpertGeometry(H, F)
    stride = pool.nbytes // E
    logits, scale = synth.router_logits(E, 900), np.ones(E, np.float32)
    x = synth.activations(H, 1, 950)[0]
    sel, w = np.zeros(K, np.int32), np.zeros(K, np.float32)
    eo, y = np.zeros((K, H), np.float32), np.zeros(H, np.float32)
    driver = ref is not None and hasattr(ref, "refdrv_moe_decode_step")
    expert_threads = min(cores, 8)
    if driver:
        scratch = np.zeros(K * (2 * F + H), np.float32)
        step = lambda: ref.refdrv_moe_decode_step(ptr(pool), stride, E, K, H, F, ptr(logits), ptr(scale), ptr(x), ptr(sel),
                                                  ptr(w), ptr(eo), ptr(y), ptr(scratch), expert_threads)
    else:
        step = lambda: oracle.orc_moe_decode_step(C.byref(g), ptr(pool), E, K, ptr(logits), ptr(scale), ptr(x), ptr(sel),
                                                  ptr(w), ptr(eo), ptr(y), expert_threads)
    steps_per_s, reps = rate(step, 1, budget_s)
    out["moe_decode_step_us"] = {"value": round(1e6 / steps_per_s, 1), "kind": "reference-constituents" if driver else "port",
                                 "cores": expert_threads, "sample": f"{reps} layer-steps"}
    # MoE prefill, grouped per expert: a 32-token sample of the 2048-token workload through salt_moe_group_execute
    T = 32
    psel, pw = synth.zipf_selection(T, E, K, 1.1, 60)
    px, py = synth.activations(H, T, 61), np.zeros((T, H), np.float32)
    if driver:
        gscratch = np.zeros(T * (2 * F + 2 * H + K * H), np.float32)
        group = lambda: ref.refdrv_moe_group(ptr(pool), stride, E, K, H, F, T, ptr(psel), ptr(pw), ptr(px), ptr(py),
                                             ptr(gscratch))
    else:
        group = lambda: oracle.orc_moe_group(C.byref(g), ptr(pool), E, K, T, ptr(psel), ptr(pw), ptr(px), ptr(py), None, cores)
    tok_per_s, reps = rate(group, T, budget_s)
    out["moe_prefill_tokens_per_s"] = {"value": round(tok_per_s, 1), "kind": "reference-constituents" if driver else "port",
                                       "cores": cores, "sample": f"{reps} passes over {T} tokens; the reference's batch "
                                       "matvec splits rows over the cores"}
    # the whole feed-forward block of a layer (port of feed_forward; matvecs and experts on `cores` threads)
    from oracle_lib import ffn_layer_struct
    weights = synth.ffn_layer(H, 2112, F, E, K, 70, pool=pool)
    layer = ffn_layer_struct(weights)
    residual = (synth.activations(H, 1, 71)[0] * 3).astype(np.float32)
    blocks_per_s, reps = rate(lambda: oracle.orc_ffn_block(C.byref(layer), ptr(residual), ptr(y), None, None, cores), 1,
                              budget_s)
    out["ffn_block_us"] = {"value": round(1e6 / blocks_per_s, 1), "kind": "port", "cores": cores,
                           "sample": f"{reps} blocks"}
    # NVFP4 8192 x 8192, batch 1: the reference's own function (single thread)
    R = Cc = 8192
    packed, fscales = synth.nvfp4_tensor(R, Cc, 40)
    fx, fy = synth.activations(Cc, 1, 41)[0], np.zeros(R, np.float32)
    xp, xs, xd = np.zeros(Cc // 2, np.uint8), np.zeros(Cc // 16, np.uint8), np.zeros(Cc, np.float32)
    fn = ref.salt_nvfp4_matvec_reference if ref is not None else oracle.orc_nvfp4_matvec
    calls_per_s, reps = rate(lambda: fn(ptr(packed), ptr(fscales), 2688.0, 64.0, R, Cc, ptr(fx), ptr(fy), ptr(xp), ptr(xs),
                                        ptr(xd)), 1, budget_s)
    out["nvfp4_8192_matvec_us"] = {"value": round(1e6 / calls_per_s, 1), "kind": "reference" if ref is not None else "port",
                                   "cores": 1, "sample": f"{reps} calls"}
    return out


def copy_leg(gpu, lib, stream, events):
    """A 512 MiB device-to-device copy: the known-size transfer that calibrates FETCH_SIZE / WRITE_SIZE."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemcpyAsync.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
    n = 512 << 20
    src, dst = gpu.DeviceBuffer(n, fill=1), gpu.DeviceBuffer(n, fill=0)
    for _ in range(3):
        assert hip.hipMemcpyAsync(dst.ptr, src.ptr, n, 3, stream) == 0
    assert lib.salt_mi355_stream_sync(stream) == 0
    return {"copy_bytes": n}


def sweep_record(lib, sweep, ms, steps, warmup):
    gbs = sweep.bytes_per_step / (ms * 1e-3) / 1e9
    launches = len(sweep.launches)
    bytes_per_launch = sweep.bytes_per_step / launches
    launch_us = ms * 1e3 / launches
    kernel = lib.salt_mi355_last_kernel().decode()
    traffic, source = TRAFFIC_FROM_PROFILE.get((kernel.split("<")[0], sweep.tokens), (None, None))
    klass = ("bit-exact kernel" if sweep.exact else
             "tolerance-class kernel (|err| <= 2^-20 sum (|q s| + 16|s| + |b|)|x| + 1e-6 per output)")
    return {
        "metric": "q4_decode_matvec_hbm_gbps", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {
            "workload": "BASELINE configs[1]: affine-Q4 group-64 decode matvec sweep, batch %d, "
                        "(K,N) in {(2816,2816),(2816,16384),(8192,2816)}, %s" % (sweep.tokens, klass),
            "instances_per_shape": [g for _, g, _ in sweep.launches],
            "launches_per_step": launches,
            "weights": "one seeded instance per shape replicated at distinct HBM addresses",
        },
        "roofline": {
            "bound": "hbm", "achieved": round(bytes_per_launch / (launch_us * 1e-6) / 1e9, 1),
            "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(bytes_per_launch / (launch_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
            "traffic": traffic, "traffic_source": source, "kernel": kernel,
            "bytes_per_launch": int(bytes_per_launch), "launch_us": round(launch_us, 2),
        },
    }


def moe_leg(gpu, synth, lib, stream, events, pool, tolerance_class):
    """MoE decode layer-step, E = 128 top-8, d_model 2816, d_ff 704.  Two layer instances (857 MB of experts) and 32
    logit vectors per layer taken in turn, so that the selection changes from step to step and the 256 MB last-level
    cache cannot hold the experts a step reads."""
    E, K, H, F = 128, 8, 2816, 704
    layers = [gpu.MoeLayer(pool, E, H, F, K) for _ in range(2)]
    logit_sets = []
    for i, layer in enumerate(layers):
        layer.tolerance_class = tolerance_class
        logit_sets.append([gpu.DeviceBuffer.from_host(synth.router_logits(E, 900 + 100 * i + k)) for k in range(32)])
        layer.scale.upload(np.ones(E, np.float32))
        layer.x.upload(synth.activations(H, 1, 950 + i)[0])
    turn = [0]

    def moe_step(st):
        for layer, sets in zip(layers, logit_sets):
            layer.logits = sets[turn[0] % len(sets)]
            if layer.enqueue(st) != 0:
                raise RuntimeError(lib.salt_mi355_last_error().decode())
        turn[0] += 1

    ms_moe = timed(lib, stream, events, moe_step, 5, 100) / len(layers)
    step_bytes = synth.moe_step_bytes(H, F, E, K)
    tag = "moe_decode_step_class_t" if tolerance_class else "moe_decode_step"
    out = {tag + "_us": round(ms_moe * 1e3, 2),
           tag + "_gbps": round(step_bytes / (ms_moe * 1e-3) / 1e9, 1),
           tag + "_hbm_frac": round(step_bytes / (ms_moe * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    out["moe_layer_tokens_per_s_class_t" if tolerance_class else "moe_layer_tokens_per_s"] = round(1e3 / ms_moe, 1)
    # the same 64 steps (32 logit vectors x 2 layers) captured once and replayed as one HIP graph: what an engine that
    # captures a token's layers would see of the launch boundaries
    if lib.salt_mi355_graph_begin(stream) == 0:
        turn[0] = 0
        for _ in range(len(logit_sets[0])):
            moe_step(stream)
        graph = lib.salt_mi355_graph_end(stream)
        if graph:
            steps_in_graph = len(logit_sets[0]) * len(layers)
            ms_g = timed(lib, stream, events, lambda st: lib.salt_mi355_graph_launch(graph, st), 2, 10) / steps_in_graph
            out[tag + "_graph_us"] = round(ms_g * 1e3, 2)
            lib.salt_mi355_graph_destroy(graph)
    return out


def nvfp4_class_t_leg(gpu, synth, lib, stream, events, w, per, packed_bytes, x, st, R, Cc, G):
    y = gpu.DeviceBuffer(G * R * 4)
    turn = [0]

    def single(s):
        g = turn[0] % G
        turn[0] += 1
        if lib.salt_mi355_nvfp4_matvec_t_dev(w.at(g * per), w.at(g * per + packed_bytes), 2688.0, 64.0, R, Cc, 1, x.ptr,
                                             y.ptr, st.ptr, s) != 0:
            raise RuntimeError(lib.salt_mi355_last_error().decode())

    ms_1 = timed(lib, stream, events, single, 5, 100)
    jobs = (gpu.Fp4Job * G)()
    for g in range(G):
        jobs[g] = gpu.Fp4Job(w.at(g * per), w.at(g * per + packed_bytes), 2688.0, x.ptr, y.at(g * R * 4), R)

    def multi(s):
        if lib.salt_mi355_nvfp4_jobs_t_dev(jobs, G, Cc, 1, 64.0, st.ptr, s) != 0:
            raise RuntimeError(lib.salt_mi355_last_error().decode())

    ms_16 = timed(lib, stream, events, multi, 3, 20)
    gbps = G * synth.nvfp4_bytes(R, Cc, 1) / (ms_16 * 1e-3) / 1e9
    return {"nvfp4_8192_class_t_matvec_us": round(ms_1 * 1e3, 2),
            "nvfp4_8192_class_t_gbps": round(synth.nvfp4_bytes(R, Cc, 1) / (ms_1 * 1e-3) / 1e9, 1),
            "nvfp4_8192_x16_class_t_one_launch_gbps": round(gbps, 1),
            "nvfp4_8192_x16_class_t_hbm_frac": round(gbps / HBM_PEAK_GBS, 4),
            "nvfp4_class_t_kernel": lib.salt_mi355_last_kernel().decode()}


def prefill_leg(gpu, synth, lib, stream, events, pool):
    """MoE prefill, 2048 tokens through one layer (E = 128, top-8, Zipf 1.1), grouped per expert, matrix cores."""
    E, K, H, F, T = 128, 8, 2816, 704, 2048
    sel, wts = synth.zipf_selection(T, E, K, 1.1, 60)
    prefill = gpu.MoePrefill(pool, E, H, F, K, T)
    prefill.sel.upload(sel); prefill.w.upload(wts); prefill.x.upload(synth.activations(H, T, 61))

    def prefill_step(s):
        if prefill.enqueue(s) != 0:
            raise RuntimeError(lib.salt_mi355_last_error().decode())

    ms_pf = timed(lib, stream, events, prefill_step, 2, 10)
    flops = 2.0 * T * K * 3 * H * F                       # useful: one pass over the weights per routed row
    # the activation travels as two exact fp16 planes, so the matrix cores execute twice the useful flops (fp16 and
    # bf16 share the dense peak)
    return {"moe_prefill_2048_us": round(ms_pf * 1e3, 1),
            "moe_prefill_tokens_per_s": round(T / (ms_pf * 1e-3), 0),
            "moe_prefill_useful_tflops": round(flops / (ms_pf * 1e-3) / 1e12, 1),
            "moe_prefill_mfma_frac": round(2 * flops / (ms_pf * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}


def nvfp4_b256_leg(gpu, synth, lib, stream, events, w, scales_at, st, R, Cc):
    """NVFP4 R x Cc, batch 256, on the matrix cores (tolerance class); the activation pass is part of the call."""
    B = 256
    xb = gpu.DeviceBuffer.from_host(synth.activations(Cc, B, 42))
    yb = gpu.DeviceBuffer(B * R * 4)
    wsb = gpu.DeviceBuffer(lib.salt_mi355_nvfp4_matmul_workspace_bytes(R, Cc, B))

    def fp4_matmul_step(s):
        if lib.salt_mi355_nvfp4_matmul_dev(w.at(0), w.at(scales_at), 2688.0, 64.0, R, Cc, B, xb.ptr, yb.ptr,
                                           st.ptr, wsb.ptr, s) != 0:
            raise RuntimeError(lib.salt_mi355_last_error().decode())

    ms_mm = timed(lib, stream, events, fp4_matmul_step, 2, 20)
    return {"nvfp4_8192_b256_matmul_us": round(ms_mm * 1e3, 2),
            "nvfp4_8192_b256_tflops": round(2.0 * R * Cc * B / (ms_mm * 1e-3) / 1e12, 1),
            "nvfp4_8192_b256_mfma_frac": round(2.0 * R * Cc * B / (ms_mm * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}


def ffn_leg(gpu, synth, lib, stream, events, pool, E, K, H, F):
    out = {}
    # the whole feed-forward block of a decoder layer for one token: pre-norms, dense FFN (2112 wide), router input,
    # 8-bit gate, top-8 of 128, routed experts, parallel combine -- bit-exact, device-resident.  32 residuals taken
    # in turn: the routing, hence the experts read, changes from block to block.
    block = gpu.FfnBlock(synth.ffn_layer(H, 2112, F, E, K, 70, pool=pool))
    residuals = [gpu.DeviceBuffer.from_host((synth.activations(H, 1, 71 + k)[0] * 3).astype(np.float32))
                 for k in range(32)]
    ffn_turn = [0]

    def ffn_step(st):
        block.residual = residuals[ffn_turn[0] % len(residuals)]
        ffn_turn[0] += 1
        if block.enqueue(st) != 0:
            raise RuntimeError(lib.salt_mi355_last_error().decode())

    ms_ffn = timed(lib, stream, events, ffn_step, 5, 100)
    if int(block.status.to_host(np.int32)[0]) != 0:
        raise RuntimeError("the feed-forward block rejected its input")
    out["ffn_block_us"] = round(ms_ffn * 1e3, 2)
    out["ffn_block_layer_tokens_per_s"] = round(1e3 / ms_ffn, 1)
    # the same block captured once and replayed as a HIP graph
    if lib.salt_mi355_graph_begin(stream) == 0:              # one residual: a graph replays fixed pointers
        ffn_step(stream)
        graph = lib.salt_mi355_graph_end(stream)
        if graph:
            ms_g = timed(lib, stream, events, lambda st: lib.salt_mi355_graph_launch(graph, st), 5, 100)
            out["ffn_block_graph_us"] = round(ms_g * 1e3, 2)
            lib.salt_mi355_graph_destroy(graph)
    return out


def abi_leg(synth, lib, pool, H, F, K):
    """The engine-facing ABI with host pointers: per-call latency of salt_gpu_q4_matvec and salt_gpu_q4_moe_chain."""
    out = {}
    # BASELINE configs[0] through the engine-facing ABI: host pointers in and out (activation upload, launch,
    # result download and a stream sync per call); a latency figure, never a throughput claim
    import ctypes as C
    R0 = C0 = 4096
    v0, s0, b0 = synth.q4_tensor(R0, C0, 0)
    blob = np.concatenate([v0.view(np.uint8), s0.view(np.uint8), b0.view(np.uint8)])
    base = blob.ctypes.data
    vp = C.c_void_p
    lib.salt_gpu_weight_resource_describe.argtypes = [C.c_uint32, C.c_uint32, vp, C.c_size_t]
    lib.salt_gpu_weight_resource_activate.argtypes = [C.c_uint32, C.c_uint32, C.c_int]
    lib.salt_gpu_weight_resource_deactivate.argtypes = [C.c_uint32, C.c_uint32]
    lib.salt_gpu_q4_matvec.argtypes = [vp, vp, vp, C.c_int, C.c_int, vp, vp]
    x0, y0 = synth.activations(C0, 1, 1)[0], np.zeros(R0, np.float32)
    if (lib.salt_gpu_init() == 0 and lib.salt_gpu_weight_resource_describe(1, 900, base, blob.nbytes) == 0
            and lib.salt_gpu_weight_resource_activate(1, 900, 2) == 0):
        def abi_call():
            if lib.salt_gpu_q4_matvec(base, base + v0.nbytes, base + v0.nbytes + s0.nbytes, R0, C0,
                                      x0.ctypes.data, y0.ctypes.data) != 0:
                raise RuntimeError(lib.salt_mi355_last_error().decode())
        def per_call_us(call, warm, reps=200):
            for _ in range(warm):
                call()
            t0 = time.perf_counter()
            for _ in range(reps):
                call()
            return round((time.perf_counter() - t0) / reps * 1e6, 1)

        out["abi_q4_matvec_4096_host_pointers_us"] = per_call_us(abi_call, 5)
        # the same call after the engine has opted into the tolerance class (salt_mi355_set_tolerance_class)
        lib.salt_mi355_set_tolerance_class(1)
        out["abi_q4_matvec_4096_host_pointers_class_t_us"] = per_call_us(abi_call, 5)
        lib.salt_mi355_set_tolerance_class(0)
        # defer mode (salt_gpu_set_defer): a hundred calls enqueued, one salt_gpu_sync at the end -- what a call costs when
        # the engine does not wait for each result
        lib.salt_gpu_set_defer.argtypes = [C.c_int]

        def deferred_us(reps=100):
            lib.salt_gpu_set_defer(1)
            for _ in range(5):
                abi_call()
            lib.salt_gpu_sync()
            t0 = time.perf_counter()
            for _ in range(reps):
                abi_call()
            lib.salt_gpu_sync()
            us = (time.perf_counter() - t0) / reps * 1e6
            lib.salt_gpu_set_defer(0)
            return round(us, 1)

        out["abi_q4_matvec_4096_deferred_us"] = deferred_us()
        lib.salt_mi355_set_tolerance_class(1)
        out["abi_q4_matvec_4096_deferred_class_t_us"] = deferred_us()
        lib.salt_mi355_set_tolerance_class(0)
        lib.salt_gpu_weight_resource_deactivate(1, 900)
        # the engine's decode call for the routed experts: salt_gpu_q4_moe_chain over eight experts, one row each
        import engine_abi
        eabi = engine_abi.bind(lib)
        if eabi.salt_gpu_expert_resource_bind(901, pool.ctypes.data, pool.nbytes) == 0:
            proj, n = synth.expert_proj_bytes(H, F), H * F
            recs = (engine_abi.MoeExpert * K)()
            for i, e8 in enumerate(range(3, 3 + 15 * K, 15)):
                at = pool.ctypes.data + e8 * 3 * proj
                for p_, name in enumerate(("gate", "up", "down")):
                    setattr(recs[i], name + "_vals", at + p_ * proj)
                    setattr(recs[i], name + "_scales", at + p_ * proj + n // 2)
                    setattr(recs[i], name + "_biases", at + p_ * proj + n // 2 + (n // 64) * 2)
                    setattr(recs[i], name + "_id", at + p_ * proj)
                recs[i].group, recs[i].resource_slot, recs[i].logical_resource_id = 1, -1, 0
            xin = np.tile(synth.activations(H, 1, 7)[0], (K, 1)).astype(np.float32)
            yout, scr = np.zeros((K, H), np.float32), np.zeros((2, K * F), np.float32)

            def chain_call():
                if eabi.salt_gpu_q4_moe_chain(recs, K, H, F, xin.ctypes.data, yout.ctypes.data, scr[0].ctypes.data,
                                              scr[1].ctypes.data, K * F) != 0:
                    raise RuntimeError(lib.salt_mi355_last_error().decode())
            out["abi_q4_moe_chain_8_experts_us"] = per_call_us(chain_call, 20)
            lib.salt_mi355_set_tolerance_class(1)
            out["abi_q4_moe_chain_8_experts_class_t_us"] = per_call_us(chain_call, 20)
            lib.salt_mi355_set_tolerance_class(0)
            eabi.salt_gpu_expert_resource_unbind(901)
    return out


def run_only(args, gpu, synth, lib, stream, events):
    """One leg on its own, for profiler runs: the kernels of that leg are the only matvec kernels in the trace."""
    if args.only == "copy":
        return copy_leg(gpu, lib, stream, events)
    if args.only in ("sweep", "sweep-exact", "sweep-b4", "sweep-b4-exact"):
        sweep = Q4Sweep(gpu, synth, tokens=4 if "b4" in args.only else 1, exact=args.only.endswith("exact"))
        ms = timed(lib, stream, events, sweep.step, args.warmup, args.steps)
        return sweep_record(lib, sweep, ms, args.steps, args.warmup)
    if args.only in ("moe", "moe-t"):
        pool = synth.expert_pool(128, 2816, 704, 7)
        return moe_leg(gpu, synth, lib, stream, events, pool, args.only == "moe-t")
    if args.only == "ffn":
        return ffn_leg(gpu, synth, lib, stream, events, synth.expert_pool(128, 2816, 704, 7), 128, 8, 2816, 704)
    if args.only == "abi":
        return abi_leg(synth, lib, synth.expert_pool(128, 2816, 704, 7), 2816, 704, 8)
    if args.only == "prefill":
        return prefill_leg(gpu, synth, lib, stream, events, synth.expert_pool(128, 2816, 704, 7))
    if args.only in ("single", "single-exact"):
        # every matrix of the decode sweep as a launch of its own (what the engine's salt_gpu_q4_matvec issues)
        sweep = Q4Sweep(gpu, synth, tokens=1, exact=args.only.endswith("exact"))
        out = {}
        for i, (R, Cc) in enumerate(SWEEP):
            ms_1 = timed(lib, stream, events, lambda st, i=i: sweep.single_launches(i, st), 1, 3) / sweep.launches[i][1]
            out[f"q4_{R}x{Cc}_single_launch_us"] = round(ms_1 * 1e3, 2)
            out[f"q4_{R}x{Cc}_kernel"] = lib.salt_mi355_last_kernel().decode()
        return out
    if args.only == "nvfp4-b256":
        R = Cc = 8192
        packed, fscales = synth.nvfp4_tensor(R, Cc, 40)
        w = gpu.DeviceBuffer(packed.nbytes + fscales.nbytes)
        w.upload(packed, 0)
        w.upload(fscales, packed.nbytes)
        st = gpu.DeviceBuffer(4, fill=0)
        return nvfp4_b256_leg(gpu, synth, lib, stream, events, w, packed.nbytes, st, R, Cc)
    if args.only == "nvfp4-t":
        R = Cc = 8192
        packed, fscales = synth.nvfp4_tensor(R, Cc, 40)
        G = 16
        per = packed.nbytes + fscales.nbytes
        w = gpu.DeviceBuffer(per * G)
        for g in range(G):
            w.upload(packed, g * per)
            w.upload(fscales, g * per + packed.nbytes)
        x = gpu.DeviceBuffer.from_host(synth.activations(Cc, 1, 41))
        st = gpu.DeviceBuffer(4, fill=0)
        return nvfp4_class_t_leg(gpu, synth, lib, stream, events, w, per, packed.nbytes, x, st, R, Cc, G)
    sys.exit("unknown leg: " + args.only)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the host baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the MoE / NVFP4 / batch-4 legs")
    ap.add_argument("--only", default="", help="run one leg: sweep | sweep-exact | sweep-b4 | sweep-b4-exact | single | single-exact | moe | moe-t | prefill | ffn | abi | nvfp4-t | nvfp4-b256 | copy")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no multi-GPU mode (run with --gpus 1)")

    from __graft_entry__ import load_package
    pkg = load_package()
    gpu, synth = pkg.lib, pkg.synth
    lib = gpu.init()
    stream = lib.salt_mi355_stream()
    events = Events(lib, stream)

    if args.only:
        print(json.dumps(run_only(args, gpu, synth, lib, stream, events)))
        return

    sweep = Q4Sweep(gpu, synth, tokens=1)
    ms = timed(lib, stream, events, sweep.step, args.warmup, args.steps)
    result = sweep_record(lib, sweep, ms, args.steps, args.warmup)

    if not args.no_extra:
        extra = {}
        extra["q4_sweep_class_t_gbps"] = result["value"]
        # configs[1] one matrix per launch (what salt_gpu_q4_matvec issues), per shape: microseconds per launch
        for i, (R, Cc) in enumerate(SWEEP):
            ms_1 = timed(lib, stream, events, lambda st, i=i: sweep.single_launches(i, st), 1, 3) / sweep.launches[i][1]
            extra[f"q4_{R}x{Cc}_single_launch_class_t_us"] = round(ms_1 * 1e3, 2)
        del sweep
        # the same sweep on the bit-exact kernel (the reference's 32-chain order and rounding points)
        sx = Q4Sweep(gpu, synth, tokens=1, exact=True)
        ms_x = timed(lib, stream, events, sx.step, args.warmup, args.steps)
        extra["q4_sweep_bit_exact_gbps"] = round(sx.bytes_per_step / (ms_x * 1e-3) / 1e9, 1)
        extra["q4_sweep_bit_exact_kernel"] = lib.salt_mi355_last_kernel().decode()
        for i, (R, Cc) in enumerate(SWEEP):
            ms_1 = timed(lib, stream, events, lambda st, i=i: sx.single_launches(i, st), 1, 3) / sx.launches[i][1]
            extra[f"q4_{R}x{Cc}_single_launch_bit_exact_us"] = round(ms_1 * 1e3, 2)
        del sx
        # batch 4 of the same sweep, both kernels
        for name, exact in (("q4_sweep_batch4_class_t_gbps", False), ("q4_sweep_batch4_bit_exact_gbps", True)):
            s4 = Q4Sweep(gpu, synth, tokens=4, exact=exact)
            ms4 = timed(lib, stream, events, s4.step, args.warmup, args.steps)
            extra[name] = round(s4.bytes_per_step / (ms4 * 1e-3) / 1e9, 1)
            del s4
        # the same batch-1 launches with every job reading one of two weight instances per shape (87 MB in all):
        # served by the 256 MB last-level cache instead of HBM
        for name, exact in (("q4_sweep_cache_warm_class_t_gbps", False), ("q4_sweep_cache_warm_bit_exact_gbps", True)):
            warm = Q4Sweep(gpu, synth, tokens=1, distinct=2, exact=exact)
            ms_w = timed(lib, stream, events, warm.step, 5, max(20, args.steps))
            extra[name] = round(warm.bytes_per_step / (ms_w * 1e-3) / 1e9, 1)
            del warm
        # MoE decode layer-step, E = 128 top-8, d_model 2816, d_ff 704: bit-exact plan and tolerance-class plan
        E, K, H, F = 128, 8, 2816, 704
        pool = synth.expert_pool(E, H, F, 7)
        extra.update(moe_leg(gpu, synth, lib, stream, events, pool, False))
        extra.update(moe_leg(gpu, synth, lib, stream, events, pool, True))
        # what the step's two launches cost with nothing in them: the same grids, workgroup sizes and LDS, empty bodies
        # (353 x 384 threads x 63 KB, then 176 x 512 threads x 101 KB: the class-T plan at this geometry)
        shape = (353, 384, 62_848, 176, 512, 100_608)
        if lib.salt_mi355_launch_skeleton_dev(*shape, stream) == 0:
            ms_sk = timed(lib, stream, events, lambda st: lib.salt_mi355_launch_skeleton_dev(*shape, st), 5, 200)
            extra["moe_launch_skeleton_us"] = round(ms_sk * 1e3, 2)
            ms_sk1 = timed(lib, stream, events, lambda st: lib.salt_mi355_launch_skeleton_dev(128, 512, 0, 0, 0, 0, st), 5, 200)
            extra["single_launch_skeleton_us"] = round(ms_sk1 * 1e3, 2)
        extra.update(ffn_leg(gpu, synth, lib, stream, events, pool, E, K, H, F))
        # BASELINE configs[0]: one 4096 x 4096 Q4 matvec per launch, batch 1, rotating through 64 weight instances (606 MB)
        R = Cc = 4096
        vals, scales, biases = synth.q4_tensor(R, Cc, 60)
        G = 64
        per = vals.nbytes + scales.nbytes + biases.nbytes
        w0 = gpu.DeviceBuffer(per * G)
        for g in range(G):
            w0.upload(vals, g * per)
            w0.upload(scales, g * per + vals.nbytes)
            w0.upload(biases, g * per + vals.nbytes + scales.nbytes)
        x0 = gpu.DeviceBuffer.from_host(synth.activations(Cc, 1, 61))
        y0 = gpu.DeviceBuffer(R * 4)

        def q4_single_step(s):
            for g in range(G):
                at = g * per
                if lib.salt_mi355_q4_matvec_dev(w0.at(at), w0.at(at + vals.nbytes), w0.at(at + vals.nbytes + scales.nbytes),
                                                R, Cc, 1, x0.ptr, y0.ptr, 0, s) != 0:
                    raise RuntimeError(lib.salt_mi355_last_error().decode())

        ms_q0 = timed(lib, stream, events, q4_single_step, 2, 10) / G
        extra["q4_4096_matvec_us"] = round(ms_q0 * 1e3, 2)
        extra["q4_4096_matvec_gbps"] = round(synth.q4_bytes(R, Cc, 1) / (ms_q0 * 1e-3) / 1e9, 1)

        def q4_single_step_t(s):
            for g in range(G):
                at = g * per
                if lib.salt_mi355_q4_matvec_t_dev(w0.at(at), w0.at(at + vals.nbytes), w0.at(at + vals.nbytes + scales.nbytes),
                                                  R, Cc, 1, x0.ptr, y0.ptr, s) != 0:
                    raise RuntimeError(lib.salt_mi355_last_error().decode())

        ms_q0t = timed(lib, stream, events, q4_single_step_t, 2, 10) / G
        extra["q4_4096_class_t_matvec_us"] = round(ms_q0t * 1e3, 2)
        extra["q4_4096_class_t_matvec_gbps"] = round(synth.q4_bytes(R, Cc, 1) / (ms_q0t * 1e-3) / 1e9, 1)
        del w0, x0, y0
        # NVFP4 8192 x 8192, batch 1, reference semantics (activation Q/DQ inside the rows' launch), 16 instances
        R = Cc = 8192
        packed, fscales = synth.nvfp4_tensor(R, Cc, 40)
        G = 16
        per = packed.nbytes + fscales.nbytes
        w = gpu.DeviceBuffer(per * G)
        for g in range(G):
            w.upload(packed, g * per)
            w.upload(fscales, g * per + packed.nbytes)
        x = gpu.DeviceBuffer.from_host(synth.activations(Cc, 1, 41))
        y, st = gpu.DeviceBuffer(R * 4), gpu.DeviceBuffer(4, fill=0)

        def fp4_step(s):
            for g in range(G):
                if lib.salt_mi355_nvfp4_matvec_qdq_dev(w.at(g * per), w.at(g * per + packed.nbytes), 2688.0, 64.0, R, Cc,
                                                       x.ptr, y.ptr, st.ptr, 0, s) != 0:
                    raise RuntimeError(lib.salt_mi355_last_error().decode())

        ms_fp4 = timed(lib, stream, events, fp4_step, 2, 10) / G
        extra["nvfp4_8192_matvec_us"] = round(ms_fp4 * 1e3, 2)
        extra["nvfp4_8192_gbps"] = round(synth.nvfp4_bytes(R, Cc, 1) / (ms_fp4 * 1e-3) / 1e9, 1)
        # the same 16 instances as ONE multi-matrix launch after one activation pass: the kernel's streaming rate
        xq = gpu.DeviceBuffer(Cc * 4)
        ys16 = gpu.DeviceBuffer(G * R * 4)
        fjobs = (gpu.Fp4Job * G)()
        for g in range(G):
            fjobs[g] = gpu.Fp4Job(w.at(g * per), w.at(g * per + packed.nbytes), 2688.0, xq.ptr, ys16.at(g * R * 4), R)

        def fp4_sweep_step(s):
            lib.salt_mi355_nvfp4_qdq_dev(x.ptr, Cc, 1, 64.0, None, None, xq.ptr, st.ptr, s)
            if lib.salt_mi355_nvfp4_jobs_dev(fjobs, G, Cc, 1, 0, s) != 0:
                raise RuntimeError(lib.salt_mi355_last_error().decode())

        ms_sw = timed(lib, stream, events, fp4_sweep_step, 2, 10)
        extra["nvfp4_8192_x16_one_launch_gbps"] = round(G * synth.nvfp4_bytes(R, Cc, 1) / (ms_sw * 1e-3) / 1e9, 1)
        # the tolerance-class kernel (exact code products per block, activation quantised inside the launch):
        # one matrix per launch, and the sixteen instances as one launch
        fp4_t = nvfp4_class_t_leg(gpu, synth, lib, stream, events, w, per, packed.nbytes, x, st, R, Cc, G)
        extra.update(fp4_t)
        del xq, ys16
        extra.update(nvfp4_b256_leg(gpu, synth, lib, stream, events, w, packed.nbytes, st, R, Cc))
        del w
        extra.update(abi_leg(synth, lib, pool, H, F, K))
        extra.update(prefill_leg(gpu, synth, lib, stream, events, pool))
        # the bf16 head (262144 x 2816, the largest matrix a decode step streams) and the 8-bit router gate
        # (128 x 2816, one unsplittable 2816-step chain per row), both bit-exact
        RH, CH = 262144, 2816
        block = (synth.rng(51).standard_normal(4096 * CH).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        head = gpu.DeviceBuffer(RH * CH * 2)
        for k in range(RH // 4096):
            head.upload(block, k * block.nbytes)
        xh = gpu.DeviceBuffer.from_host(synth.activations(CH, 1, 52))
        yh = gpu.DeviceBuffer(RH * 4)

        def head_step(s):
            if lib.salt_mi355_bf16_matvec_dev(head.ptr, RH, CH, 1, xh.ptr, None, yh.ptr, s) != 0:
                raise RuntimeError(lib.salt_mi355_last_error().decode())

        ms_h = timed(lib, stream, events, head_step, 2, 20)
        extra["bf16_head_262144x2816_us"] = round(ms_h * 1e3, 1)
        extra["bf16_head_gbps"] = round((RH * CH * 2 + RH * 4 + CH * 4) / (ms_h * 1e-3) / 1e9, 1)
        extra["bf16_head_hbm_frac"] = round((RH * CH * 2 + RH * 4 + CH * 4) / (ms_h * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
        del head, yh
        RG = 128
        gv = gpu.DeviceBuffer.from_host(synth.rng(53).integers(0, 256, RG * CH, dtype=np.uint8))
        gs = gpu.DeviceBuffer.from_host(np.full(RG * CH // 64, 0x3C00, np.uint16))
        yg = gpu.DeviceBuffer(RG * 4)

        def gate_step(s):
            if lib.salt_mi355_q8_matvec_dev(gv.ptr, gs.ptr, gs.ptr, RG, CH, 1, xh.ptr, yg.ptr, s) != 0:
                raise RuntimeError(lib.salt_mi355_last_error().decode())

        extra["q8_router_gate_128x2816_us"] = round(timed(lib, stream, events, gate_step, 5, 100) * 1e3, 2)
        result["extra"] = extra

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(synth)
        if not args.no_extra:
            result["cpu_baseline"]["other_configs"] = cpu_other_configs(synth, pool, result["cpu_baseline"]["cores"])
    print(json.dumps(result))


if __name__ == "__main__":
    main()
