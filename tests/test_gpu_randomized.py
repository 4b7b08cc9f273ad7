"""Seeded random shapes through the device entry points, bit for bit against the CPU checker: matvecs of every format
with ragged rows, odd column counts, offsets and batch sizes; router selections with ties; MoE decode steps at random
geometries, including more experts than the fused prologue holds and a single selected expert."""
import ctypes as C

import numpy as np
import pytest

from golden import cases
from oracle_lib import ExpertGeometry, bits, host_threads, ptr
from q4_bounds import check as check_class_t

pytestmark = pytest.mark.gpu
synth = cases.synth


@pytest.fixture(scope="module")
def gpu(pkg):
    pkg.lib.init()
    return pkg.lib


def q4_want(oracle, vals, scales, biases, R, Cc, xs):
    ys = np.zeros((xs.shape[0], R), np.float32)
    for t in range(xs.shape[0]):
        assert oracle.orc_q4_matvec_threads(ptr(vals), ptr(scales), ptr(biases), R, Cc, ptr(np.ascontiguousarray(xs[t])),
                                            ptr(ys[t]), host_threads()) == 0
    return ys


@pytest.mark.parametrize("stream_seed", [1, 2])
def test_random_matvecs_and_router(gpu, oracle, stream_seed):
    rng = np.random.default_rng(stream_seed)
    for case in range(150):
        kind = int(rng.integers(0, 5))
        seed = int(rng.integers(1, 1 << 30))
        if kind == 0:
            R = int(rng.integers(1, 400)); Cc = 64 * int(rng.integers(1, 64)); B = int(rng.integers(1, 7))
            chains = int(rng.choice([0, 8, 4, 2]))
            if rng.random() < 0.2:
                Cc = int(rng.integers(1, 300)); chains = 0
            pad = (-(R * Cc)) % 64
            vals, scales, biases = synth.q4_tensor(1, R * Cc + pad, seed) if pad or Cc % 64 else synth.q4_tensor(R, Cc, seed)
            xs = synth.activations(Cc, B, seed + 1)
            off = int(rng.choice([0, 0, 4, 8, 12])) if Cc % 64 == 0 else 0
            print("q4", R, Cc, B, chains, off, seed, flush=True)
            got = gpu.q4_matvec(vals, scales, biases, R, Cc, xs, chains, value_offset=off)
            assert np.array_equal(bits(got), bits(q4_want(oracle, vals, scales, biases, R, Cc, xs)))
        elif kind == 1:
            R = int(rng.integers(1, 300)); Cc = 32 * int(rng.integers(1, 128)); B = int(rng.integers(1, 5))
            chains = int(rng.choice([0, 8, 4, 2]))
            packed, fscales = synth.nvfp4_tensor(R, Cc, seed)
            xs = synth.activations(Cc, B, seed + 1)
            div = float(rng.choice([1.0, 2688.0, 0.37]))
            print("nvfp4", R, Cc, B, chains, div, seed, flush=True)
            st, y = gpu.nvfp4_matvec(packed, fscales, div, R, Cc, xs, 64.0, chains)
            want = np.zeros((B, R), np.float32)
            for t in range(B):
                scratch = (np.zeros(Cc // 2, np.uint8), np.zeros(Cc // 16, np.uint8), np.zeros(Cc, np.float32))
                assert oracle.orc_nvfp4_matvec(ptr(packed), ptr(fscales), div, 64.0, R, Cc, ptr(np.ascontiguousarray(xs[t])),
                                               ptr(want[t]), ptr(scratch[0]), ptr(scratch[1]), ptr(scratch[2])) == 0
            assert st == 0 and np.array_equal(bits(y), bits(want))
        elif kind == 2:
            R = int(rng.integers(1, 300)); Cc = 64 * int(rng.integers(1, 80)); B = int(rng.integers(1, 4))
            if rng.random() < 0.2:
                Cc = int(rng.integers(1, 200))
            pad = (-(R * Cc)) % 64
            vals, scales, biases = synth.q8_tensor(1, R * Cc + pad, seed) if pad or Cc % 64 else synth.q8_tensor(R, Cc, seed)
            xs = synth.activations(Cc, B, seed + 1)
            print("q8", R, Cc, B, seed, flush=True)
            got = gpu.q8_matvec(vals, scales, biases, R, Cc, xs)
            want = np.zeros((B, R), np.float32)
            for t in range(B):
                oracle.orc_q8_matvec(ptr(vals), ptr(scales), ptr(biases), R, Cc, ptr(np.ascontiguousarray(xs[t])), ptr(want[t]))
            assert np.array_equal(bits(got), bits(want))
        elif kind == 3:
            R = int(rng.integers(1, 600)); Cc = int(rng.integers(1, 400)) * int(rng.choice([1, 8])); B = int(rng.integers(1, 6))
            W = (synth.rng(seed).standard_normal(R * Cc).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
            xs = synth.activations(Cc, B, seed + 1)
            bias = synth.activations(R, 1, seed + 2)[0] if rng.random() < 0.5 else None
            print("bf16", R, Cc, B, bias is not None, seed, flush=True)
            got = gpu.bf16_matvec(W, R, Cc, xs, bias)
            want = np.zeros((B, R), np.float32)
            for t in range(B):
                oracle.orc_bf16_matvec(ptr(W), R, Cc, ptr(np.ascontiguousarray(xs[t])), ptr(bias) if bias is not None else None,
                                       ptr(want[t]))
            assert np.array_equal(bits(got), bits(want))
        else:
            E = int(rng.integers(2, 513)); K = int(rng.integers(1, min(E, 16) + 1))
            logits = synth.router_logits(E, seed)
            if rng.random() < 0.3:
                logits[rng.integers(0, E, 5)] = logits[0]                 # ties
            scale = synth.rng(seed + 1).uniform(0.5, 2.0, E).astype(np.float32)
            by_id = bool(rng.integers(0, 2))
            print("router", E, K, by_id, seed, flush=True)
            st, sel, w = gpu.router_topk(logits, scale, K, by_id)
            osel = np.zeros(K, np.int32); ow = np.zeros(K, np.float32)
            assert oracle.orc_router_topk(ptr(logits), ptr(scale), E, K, ptr(osel), ptr(ow)) == 0
            if by_id:
                oracle.orc_sort_selection(ptr(osel), ptr(ow), K)
            assert st == 0 and np.array_equal(sel, osel) and np.array_equal(bits(w), bits(ow))


def test_random_moe_decode_steps(gpu, oracle):
    rng = np.random.default_rng(11)
    for case in range(14):
        E = int(rng.integers(2, 200)); K = int(rng.integers(1, min(E, 16) + 1))
        H = 64 * int(rng.integers(1, 24)); F = 64 * int(rng.integers(1, 12))
        if case % 5 == 4:
            E = int(rng.integers(513, 700))                               # beyond the fused prologue: five launches
        if case == 9:
            K = 1
        seed = int(rng.integers(1, 1 << 30))
        header = int(rng.choice([0, 24]))
        print("moe", E, K, H, F, header, seed, flush=True)
        pool = synth.expert_pool(E, H, F, seed)
        layer = gpu.MoeLayer(pool, E, H, F, K, header_bytes=header)
        g = ExpertGeometry(H, F)
        scale = synth.rng(seed + 1).uniform(0.5, 2.0, E).astype(np.float32)
        for it in range(2):
            logits = synth.router_logits(E, seed + 2 + it); x = synth.activations(H, 1, seed + 5 + it)[0]
            st, sel, w, eo, y = layer.step(logits, scale, x)
            osel = np.zeros(K, np.int32); ow = np.zeros(K, np.float32)
            oeo = np.zeros((K, H), np.float32); oy = np.zeros(H, np.float32)
            assert oracle.orc_moe_decode_step(C.byref(g), ptr(pool), E, K, ptr(logits), ptr(scale), ptr(x), ptr(osel),
                                              ptr(ow), ptr(oeo), ptr(oy), host_threads()) == 0
            assert st == 0 and np.array_equal(sel, osel) and np.array_equal(bits(w), bits(ow))
            assert np.array_equal(bits(eo), bits(oeo)) and np.array_equal(bits(y), bits(oy))
        del layer


@pytest.mark.parametrize("stream_seed", [11, 12])
def test_random_tolerance_class_launches(gpu, oracle, stream_seed):
    """salt_mi355_q4_jobs_t_dev at random shapes: 512..8192 columns, 1..9 tokens, 1..40 jobs of ragged row counts,
    tensors at 0 / 4 / 8 bytes past a multiple of 16, with and without biases; every sampled job inside the stated
    bound against the CPU checker."""
    lib = gpu.init()
    rng = np.random.default_rng(stream_seed)
    kernels = set()
    for case in range(40):
        Cc = 64 * int(rng.integers(8, 129))
        tokens = int(rng.integers(1, 10))
        njobs = int(rng.choice([1, 1, 2, 3, 7, 17, 40]))
        budget = 6_000_000 // Cc                                  # rows in the launch: bounds the checker's time
        rows = [int(rng.integers(1, max(2, min(3000, 2 * budget // njobs)))) for _ in range(njobs)]
        seed = int(rng.integers(1, 1 << 30))
        offset = int(rng.choice([0, 4, 8]))
        with_bias = bool(rng.random() < 0.8)
        top = max(rows)
        tensors = [synth.q4_tensor(top, Cc, seed + k) for k in range(min(njobs, 3))]
        dev = []
        for vals, scales, biases in tensors:
            dv = gpu.DeviceBuffer(vals.nbytes + offset + 16, fill=0)
            dv.upload(vals, offset)
            dev.append((dv, gpu.DeviceBuffer.from_host(scales), gpu.DeviceBuffer.from_host(biases)))
        xs = [synth.activations(Cc, tokens, seed + 10 + j) for j in range(njobs)]
        dxs = [gpu.DeviceBuffer.from_host(x) for x in xs]
        dys = [gpu.DeviceBuffer(tokens * R * 4, fill=0xFF) for R in rows]
        jobs = (gpu.Q4Job * njobs)()
        for j, R in enumerate(rows):
            dv, ds, db = dev[j % len(dev)]
            jobs[j] = gpu.Q4Job(dv.at(offset), ds.ptr, db.ptr if with_bias else None, dxs[j].ptr, dys[j].ptr, R)
        print("class T", Cc, tokens, njobs, sum(rows), offset, with_bias, seed, flush=True)
        stream = lib.salt_mi355_stream()
        gpu.check(lib.salt_mi355_q4_jobs_t_dev(jobs, njobs, Cc, tokens, stream), "q4_jobs_t_dev")
        gpu.check(lib.salt_mi355_stream_sync(stream), "sync")
        kernels.add(lib.salt_mi355_last_kernel().decode())
        for j in sorted({0, njobs // 2, njobs - 1}):
            vals, scales, biases = tensors[j % len(tensors)]
            R = rows[j]
            v, s_, b = vals[:R * Cc // 8], scales[:R * Cc // 64], (biases[:R * Cc // 64] if with_bias else None)
            got = dys[j].to_host(np.float32).reshape(tokens, R)
            want = q4_want(oracle, v, s_, b, R, Cc, xs[j])
            check_class_t(got, want, v, s_, b, R, Cc, xs[j])
    print("kernels reached:", sorted(kernels), flush=True)


def test_random_tolerance_class_launches_of_many_blocks(gpu, oracle):
    """The same entry point at launches of at least 2048 blocks, which the sixteen-row kernel serves: 24..70 jobs of
    ragged row counts, 1..9 tokens (passes inside one launch beyond four, two column windows for wide rows at three or
    four), three sampled jobs per launch inside the stated bound."""
    lib = gpu.init()
    rng = np.random.default_rng(21)
    kernels = set()
    for case in range(10):
        Cc = 64 * int(rng.integers(8, 129))
        tokens = int(rng.integers(1, 10))
        njobs = int(rng.choice([24, 33, 40, 70]))
        lo = 70000 // njobs
        rows = [int(rng.integers(lo, lo + 1500)) for _ in range(njobs)]
        seed = int(rng.integers(1, 1 << 30))
        offset = int(rng.choice([0, 4, 8]))
        with_bias = bool(rng.random() < 0.8)
        tensors = [synth.q4_tensor(max(rows), Cc, seed + k) for k in range(2)]
        dev = []
        for vals, scales, biases in tensors:
            dv = gpu.DeviceBuffer(vals.nbytes + offset + 16, fill=0)
            dv.upload(vals, offset)
            dev.append((dv, gpu.DeviceBuffer.from_host(scales), gpu.DeviceBuffer.from_host(biases)))
        xs = [synth.activations(Cc, tokens, seed + 10 + (j % 5)) for j in range(njobs)]
        dxs = [gpu.DeviceBuffer.from_host(x) for x in xs]
        dys = [gpu.DeviceBuffer(tokens * R * 4, fill=0xFF) for R in rows]
        jobs = (gpu.Q4Job * njobs)()
        for j, R in enumerate(rows):
            dv, ds, db = dev[j % len(dev)]
            jobs[j] = gpu.Q4Job(dv.at(offset), ds.ptr, db.ptr if with_bias else None, dxs[j].ptr, dys[j].ptr, R)
        print("class T, many blocks", Cc, tokens, njobs, sum(rows), offset, with_bias, seed, flush=True)
        stream = lib.salt_mi355_stream()
        gpu.check(lib.salt_mi355_q4_jobs_t_dev(jobs, njobs, Cc, tokens, stream), "q4_jobs_t_dev")
        gpu.check(lib.salt_mi355_stream_sync(stream), "sync")
        kernels.add(lib.salt_mi355_last_kernel().decode())
        for j in sorted({0, njobs // 2, njobs - 1}):
            vals, scales, biases = tensors[j % len(tensors)]
            R = rows[j]
            v, s_, b = vals[:R * Cc // 8], scales[:R * Cc // 64], (biases[:R * Cc // 64] if with_bias else None)
            got = dys[j].to_host(np.float32).reshape(tokens, R)
            check_class_t(got, q4_want(oracle, v, s_, b, R, Cc, xs[j]), v, s_, b, R, Cc, xs[j])
        del dev, dxs, dys
    print("kernels reached:", sorted(kernels), flush=True)
    assert all(k.startswith("q4_dot16_kernel<") for k in kernels)
