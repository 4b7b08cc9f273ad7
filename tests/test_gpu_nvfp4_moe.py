"""NVFP4, router and MoE decode step on the MI355X through the C ABI,
bit-for-bit against the CPU checker and the committed reference fixtures."""
import ctypes as C

import numpy as np
import pytest

from golden import cases
from oracle_lib import ExpertGeometry, bits, host_threads, ptr

pytestmark = pytest.mark.gpu
synth = cases.synth


@pytest.fixture(scope="module")
def gpu(pkg):
    pkg.lib.init()
    return pkg.lib


def oracle_qdq(oracle, x, g):
    Cc = x.shape[-1]
    flat = x.reshape(-1, Cc)
    p = np.zeros((flat.shape[0], Cc // 2), np.uint8); s = np.zeros((flat.shape[0], Cc // 16), np.uint8)
    d = np.zeros_like(flat)
    rc = 0
    for t in range(flat.shape[0]):
        rc |= oracle.orc_nvfp4_qdq(ptr(np.ascontiguousarray(flat[t])), Cc, g, ptr(p[t]), ptr(s[t]), ptr(d[t]))
    return rc, p.ravel(), s.ravel(), d.reshape(x.shape)


@pytest.mark.parametrize("g", [64.0, 2688.0, 0.37, 1.0])
def test_qdq_matches_checker(gpu, oracle, g):
    print("qdq g", g, flush=True)
    x = synth.activations(2048, 3, int(g * 10) + 1)
    x[0, 32:48] = 0; x[1, 5] = 300.0; x[2, 100] = 1e-25; x[2, 101] = -0.0
    # exact decision boundaries of both encoders
    x[1, 64:80] = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, -0.25, -0.75, -1.25, -1.75, -2.5, -3.5,
                            -5.0, -6.0], np.float32)
    st, p, s, d = gpu.nvfp4_qdq(x, g)
    rc, op, os_, od = oracle_qdq(oracle, x, g)
    assert st == 0 and rc == 0
    assert np.array_equal(p, op) and np.array_equal(s, os_) and np.array_equal(bits(d), bits(od))


def test_qdq_reference_fixtures_and_rejection(gpu):
    fx = cases.load("nvfp4.npz")
    for tag, g, seed in cases.NVFP4_QDQ_CASES:
        x = cases.nvfp4_qdq_input(tag, seed)
        st, p, s, d = gpu.nvfp4_qdq(x, g)
        assert st == 0 and np.array_equal(p, fx[f"qdq_{tag}.packed"]) and np.array_equal(s, fx[f"qdq_{tag}.scales"])
        assert np.array_equal(bits(d), fx[f"qdq_{tag}.dequant_bits"])
    bad = synth.activations(256, 1, 3)[0]; bad[77] = np.inf
    assert gpu.nvfp4_qdq(bad, 64.0)[0] == -1
    bad[77] = np.nan
    assert gpu.nvfp4_qdq(bad, 64.0)[0] == -1
    lib = gpu.load()
    buf = gpu.DeviceBuffer(4096)
    assert lib.salt_mi355_nvfp4_qdq_dev(buf.ptr, 24, 1, 64.0, None, None, buf.ptr, buf.ptr, None) == -1
    assert lib.salt_mi355_nvfp4_qdq_dev(buf.ptr, 32, 1, 0.0, None, None, buf.ptr, buf.ptr, None) == -1


@pytest.mark.parametrize("chains", [8, 4, 2])
@pytest.mark.parametrize("R,Cc,B,divisor", [(64, 64, 1, 1.0), (96, 2816, 2, 2688.0), (130, 704, 4, 3.0),
                                            (65, 8192, 1, 0.5), (1, 32, 1, 1.0), (70, 96, 3, 2688.0)])
def test_matvec_matches_checker(gpu, oracle, R, Cc, B, divisor, chains):
    print(f"nvfp4 R={R} C={Cc} B={B} chains={chains}", flush=True)
    packed, scales = synth.nvfp4_tensor(R, Cc, R + Cc)
    xs = synth.activations(Cc, B, R * 3 + B)
    st, got = gpu.nvfp4_matvec(packed, scales, divisor, R, Cc, xs, 64.0, chains)
    want = np.zeros((B, R), np.float32)
    for t in range(B):
        xp = np.zeros(Cc // 2, np.uint8); xsc = np.zeros(Cc // 16, np.uint8); xd = np.zeros(Cc, np.float32)
        assert oracle.orc_nvfp4_matvec(ptr(packed), ptr(scales), divisor, 64.0, R, Cc, ptr(xs[t]), ptr(want[t]),
                                       ptr(xp), ptr(xsc), ptr(xd)) == 0
    assert st == 0 and np.array_equal(bits(got), bits(want))
    # weights-only variant: the activation is used as given
    st, got = gpu.nvfp4_matvec(packed, scales, divisor, R, Cc, xs, None, chains)
    for t in range(B):
        assert oracle.orc_nvfp4_matvec_weights_only(ptr(packed), ptr(scales), divisor, R, Cc, ptr(xs[t]),
                                                    ptr(want[t])) == 0
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("chains", [0, 8, 4, 2])
@pytest.mark.parametrize("R,Cc,g", [(64, 64, 64.0), (130, 2816, 8.0), (65, 8192, 64.0), (1, 32, 1.0), (704, 704, 100.0)])
def test_matvec_with_activation_pass_in_one_launch(gpu, oracle, R, Cc, g, chains):
    print(f"nvfp4 one launch R={R} C={Cc} g={g} chains={chains}", flush=True)
    packed, scales = synth.nvfp4_tensor(R, Cc, R * 7 + Cc)
    x = synth.activations(Cc, 1, R + 11)[0]
    x[:3] = [0.0, -0.0, 1e-30]
    want = np.zeros(R, np.float32)
    xp = np.zeros(Cc // 2, np.uint8); xsc = np.zeros(Cc // 16, np.uint8); xd = np.zeros(Cc, np.float32)
    assert oracle.orc_nvfp4_matvec(ptr(packed), ptr(scales), 2688.0, g, R, Cc, ptr(x), ptr(want), ptr(xp), ptr(xsc),
                                   ptr(xd)) == 0
    st, got = gpu.nvfp4_matvec_one_launch(packed, scales, 2688.0, R, Cc, x, g, chains)
    assert st == 0 and np.array_equal(bits(got), bits(want))
    bad = x.copy(); bad[Cc - 1] = np.inf
    st, got = gpu.nvfp4_matvec_one_launch(packed, scales, 2688.0, R, Cc, bad, g, chains)
    assert st == -1 and (got.view(np.uint32) == 0xFFFFFFFF).all()


@pytest.mark.parametrize("tokens", [1, 3, 6])
def test_many_matrices_in_one_launch(gpu, oracle, tokens):
    print(f"nvfp4 jobs tokens={tokens}", flush=True)
    Cc = 704
    rows = [64, 130, 1, 700, 65]
    lib = gpu.init()
    stream = lib.salt_mi355_stream()
    jobs = (gpu.Fp4Job * len(rows))()
    keep, wants = [], []
    for j, R in enumerate(rows):
        packed, scales = synth.nvfp4_tensor(R, Cc, 50 + j)
        xs = synth.activations(Cc, tokens, 60 + j)
        divisor = [1.0, 2688.0, -3.0, 0.5, 7.0][j]
        want = np.zeros((tokens, R), np.float32)
        for t in range(tokens):
            assert oracle.orc_nvfp4_matvec_weights_only(ptr(packed), ptr(scales), divisor, R, Cc, ptr(xs[t]),
                                                        ptr(want[t])) == 0
        dp, ds, dx = (gpu.DeviceBuffer.from_host(a) for a in (packed, scales, xs))
        dy = gpu.DeviceBuffer(tokens * R * 4, fill=0xFF)
        keep.append((dp, ds, dx, dy)); wants.append(want)
        jobs[j] = gpu.Fp4Job(dp.ptr, ds.ptr, divisor, dx.ptr, dy.ptr, R)
    assert lib.salt_mi355_nvfp4_jobs_dev(jobs, len(rows), Cc, tokens, 0, stream) == 0
    assert lib.salt_mi355_stream_sync(stream) == 0
    for (dp, ds, dx, dy), want in zip(keep, wants):
        assert np.array_equal(bits(dy.to_host(np.float32).reshape(want.shape)), bits(want))
    jobs[1].stored_divisor = 0.0
    assert lib.salt_mi355_nvfp4_jobs_dev(jobs, len(rows), Cc, tokens, 0, stream) == -1


def test_matvec_nan_scale_codes_and_negative_divisor(gpu, oracle):
    R, Cc = 64, 128
    packed, scales = synth.nvfp4_tensor(R, Cc, 5)
    scales = scales.copy(); scales[3] = 0x7f; scales[9] = 0x00; scales[10] = 0x80; scales[11] = 0xfe
    xs = synth.activations(Cc, 1, 6)
    st, got = gpu.nvfp4_matvec(packed, scales, -7.0, R, Cc, xs, None)
    want = np.zeros(R, np.float32)
    assert oracle.orc_nvfp4_matvec_weights_only(ptr(packed), ptr(scales), -7.0, R, Cc, ptr(xs[0]), ptr(want)) == 0
    same = (bits(got[0]) == bits(want)) | (np.isnan(got[0]) & np.isnan(want))
    assert same.all() and np.isnan(want[0])


@pytest.mark.parametrize("case", cases.NVFP4_MATVEC_CASES, ids=lambda c: c[0])
def test_matvec_reference_fixtures(gpu, case):
    name, R, Cc, wseed, xseed, divisor, g = case
    fx = cases.load("nvfp4.npz")
    packed, scales = synth.nvfp4_tensor(R, Cc, wseed)
    x = synth.activations(Cc, 1, xseed)
    assert cases.digest(packed, scales, x[0]) == str(fx[name + ".digest"])
    st, got = gpu.nvfp4_matvec(packed, scales, divisor, R, Cc, x, g)
    assert st == 0 and np.array_equal(bits(got[0]), fx[name + ".y_bits"])


def test_router_reference_fixtures(gpu):
    fx = cases.load("router.npz")
    logits = fx["logits_bits"].view(np.float32); scale = fx["scale_bits"].view(np.float32)
    K = fx["selected"].shape[1]
    for i in range(logits.shape[0]):
        st, sel, w = gpu.router_topk(logits[i], scale[i], K)
        assert st == 0 and np.array_equal(sel, fx["selected"][i]) and np.array_equal(bits(w), fx["weight_bits"][i]), i
        st, sel2, w2 = gpu.router_topk(logits[i], scale[i], K, sorted_by_id=True)
        order = np.argsort(fx["selected"][i], kind="stable")
        assert np.array_equal(sel2, fx["selected"][i][order]) and np.array_equal(bits(w2), fx["weight_bits"][i][order])


@pytest.mark.parametrize("E,K,seed", [(8, 2, 1), (5, 5, 2), (64, 6, 3), (200, 9, 4), (1024, 64, 5), (1, 1, 6)])
def test_router_matches_checker_and_rejects(gpu, oracle, E, K, seed):
    g = synth.rng(seed)
    logits = g.standard_normal(E).astype(np.float32)
    if seed % 2:
        logits = (np.round(logits * 2) / 2).astype(np.float32)
    scale = g.uniform(0.25, 4, E).astype(np.float32)
    sel = np.zeros(K, np.int32); w = np.zeros(K, np.float32)
    assert oracle.orc_router_topk(ptr(logits), ptr(scale), E, K, ptr(sel), ptr(w)) == 0
    st, gsel, gw = gpu.router_topk(logits, scale, K)
    assert st == 0 and np.array_equal(gsel, sel) and np.array_equal(bits(gw), bits(w))
    bad = logits.copy(); bad[E // 2] = np.nan
    st, gsel, gw = gpu.router_topk(bad, scale, K)
    assert st == -1 and (gsel.view(np.uint32) == 0xEEEEEEEE).all() and (gw.view(np.uint32) == 0xEEEEEEEE).all()
    bad = scale.copy(); bad[0] = np.inf
    assert gpu.router_topk(logits, bad, K)[0] == -1


def test_activation_and_reduce_match_checker(gpu, oracle):
    lib = gpu.load()
    fx = cases.load("bitmath.npz")
    x = fx["x_bits"].view(np.float32).copy()
    x = x[np.isfinite(x)]
    up = synth.activations(x.size, 1, 9)[0]
    dg, du, da = gpu.DeviceBuffer.from_host(x), gpu.DeviceBuffer.from_host(up), gpu.DeviceBuffer(x.size * 4)
    stream = lib.salt_mi355_stream()
    assert lib.salt_mi355_moe_activate_dev(dg.ptr, du.ptr, da.ptr, x.size, stream) == 0
    assert lib.salt_mi355_stream_sync(stream) == 0
    want = np.array([np.float32(oracle.orc_gelu_tanh(float(a))) * b for a, b in zip(x, up)], np.float32)
    assert np.array_equal(bits(da.to_host(np.float32)), bits(want))
    # gelu alone against the reference fixture: up = 1
    du.upload(np.ones(x.size, np.float32))
    assert lib.salt_mi355_moe_activate_dev(dg.ptr, du.ptr, da.ptr, x.size, stream) == 0
    assert lib.salt_mi355_stream_sync(stream) == 0
    keep = np.isfinite(fx["x_bits"].view(np.float32))
    assert np.array_equal(bits(da.to_host(np.float32)), fx["gelu_bits"][keep])
    K, H = 5, 300
    eo = synth.activations(H, K, 10); w = synth.activations(K, 1, 11)[0]
    de, dw, do = gpu.DeviceBuffer.from_host(eo), gpu.DeviceBuffer.from_host(w), gpu.DeviceBuffer(H * 4)
    assert lib.salt_mi355_moe_reduce_dev(de.ptr, dw.ptr, K, H, do.ptr, stream) == 0
    assert lib.salt_mi355_stream_sync(stream) == 0
    acc = np.zeros(H, np.float32)
    for i in range(K):
        acc = (acc + (eo[i] * w[i]).astype(np.float32)).astype(np.float32)
    assert np.array_equal(bits(do.to_host(np.float32)), bits(acc))


@pytest.mark.parametrize("njobs,Cc,rows", [(1, 704, 2816), (8, 704, 2816), (20, 64, 130), (3, 4096, 65), (16, 1088, 200)])
def test_activated_down_jobs(gpu, oracle, pkg, njobs, Cc, rows):
    """Down projections whose activation row gelu_tanh(gate) * up is computed in the launch's prologue: one record, inline
    records and a device table; bit for bit the activation kernel followed by the plain multi-job launch."""
    print("activated jobs", njobs, Cc, rows, flush=True)
    lib = gpu.load()
    gate = (synth.activations(Cc, njobs, 61) * 2).astype(np.float32)
    up = synth.activations(Cc, njobs, 62)
    both = gpu.DeviceBuffer.from_host(np.concatenate([gate.ravel(), np.zeros(32, np.float32), up.ravel()]))
    up_offset = gate.size + 32
    hold, jobs, want = [], (pkg.lib.Q4Job * njobs)(), []
    for j in range(njobs):
        vals, scales, biases = synth.q4_tensor(rows, Cc, 700 + j)
        bufs = [pkg.lib.DeviceBuffer.from_host(a) for a in (vals, scales, biases)]
        out = pkg.lib.DeviceBuffer(rows * 4, fill=0xFF)
        hold.append((bufs, out))
        jobs[j] = pkg.lib.Q4Job(bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, both.at(j * Cc * 4), out.ptr, rows)
        act = np.array([np.float32(oracle.orc_gelu_tanh(float(a))) * b for a, b in zip(gate[j], up[j])], np.float32)
        y = np.zeros(rows, np.float32)
        assert oracle.orc_q4_matvec_threads(ptr(vals), ptr(scales), ptr(biases), rows, Cc, ptr(act), ptr(y), host_threads()) == 0
        want.append(y)
    stream = lib.salt_mi355_stream()
    assert lib.salt_mi355_q4_jobs_activated_dev(jobs, njobs, Cc, up_offset, stream) == 0, lib.salt_mi355_last_error()
    assert lib.salt_mi355_stream_sync(stream) == 0
    for j in range(njobs):
        assert np.array_equal(bits(hold[j][1].to_host(np.float32)), bits(want[j])), j
    # column counts the prologue does not hold, or that are no multiple of 64
    assert lib.salt_mi355_q4_jobs_activated_dev(jobs, njobs, 4160, up_offset, stream) == -1
    assert lib.salt_mi355_q4_jobs_activated_dev(jobs, njobs, 100, up_offset, stream) == -1


@pytest.mark.parametrize("case", cases.MOE_CASES, ids=lambda c: c[0])
def test_moe_decode_step_reference_fixtures(gpu, case):
    name, E, K, H, F, pseed, lseed, xseed = case
    print("moe fixture", name, flush=True)
    fx = cases.load("moe_decode.npz")
    pool, logits, scale, x = cases.moe_case_inputs(E, H, F, pseed, lseed, xseed)
    assert cases.pool_digest(pool, logits, x) == str(fx[name + ".digest"])
    layer = gpu.MoeLayer(pool, E, H, F, K)
    st, sel, w, eo, y = layer.step(logits, scale, x)
    assert st == 0 and np.array_equal(sel, fx[name + ".selected"]) and np.array_equal(bits(w), fx[name + ".weight_bits"])
    assert np.array_equal(bits(eo), fx[name + ".expert_out_bits"])
    assert np.array_equal(bits(y), fx[name + ".y_bits"])


def test_moe_decode_step_fresh_logits_and_rejection(gpu, oracle):
    E, K, H, F = 16, 8, 2816, 704
    pool = synth.expert_pool(E, H, F, 31)
    layer = gpu.MoeLayer(pool, E, H, F, K)
    g = ExpertGeometry(H, F)
    scale = synth.rng(1).uniform(0.5, 2.0, E).astype(np.float32)
    for it in range(3):
        logits = synth.router_logits(E, 700 + it); x = synth.activations(H, 1, 800 + it)[0]
        st, sel, w, eo, y = layer.step(logits, scale, x)
        osel = np.zeros(K, np.int32); ow = np.zeros(K, np.float32)
        oeo = np.zeros((K, H), np.float32); oy = np.zeros(H, np.float32)
        assert oracle.orc_moe_decode_step(C.byref(g), ptr(pool), E, K, ptr(logits), ptr(scale), ptr(x), ptr(osel),
                                          ptr(ow), ptr(oeo), ptr(oy), host_threads()) == 0
        assert st == 0 and np.array_equal(sel, osel) and np.array_equal(bits(w), bits(ow))
        assert np.array_equal(bits(eo), bits(oeo)) and np.array_equal(bits(y), bits(oy))
    logits = synth.router_logits(E, 1).copy(); logits[3] = np.inf
    assert layer.step(logits, scale, x)[0] == -1
    # many steps in a row on one workspace, each checked against the sum of its own expert outputs in place order
    for it in range(40):
        logits = synth.router_logits(E, 900 + it); x = synth.activations(H, 1, 950 + it)[0]
        st, sel, w, eo, y = layer.step(logits, scale, x)
        assert st == 0
        acc = np.zeros(H, np.float32)
        for i in range(K):
            acc = (acc + (eo[i] * w[i]).astype(np.float32)).astype(np.float32)
        assert np.array_equal(bits(y), bits(acc)), it


@pytest.mark.parametrize("tolerance_class", [False, True], ids=["bit-exact", "class-t"])
def test_moe_decode_step_replayed_as_a_graph(gpu, oracle, tolerance_class):
    """Four consecutive steps captured once and replayed with fresh inputs (kernels only; the bit-exact plan's tile
    counters are zeroed by its own first launch, so a replay needs nothing from the host): every replay equals the
    eager step on the same inputs, with eager work and synchronisations between the replays."""
    print("moe step graph replay", "class T" if tolerance_class else "bit-exact", flush=True)
    E, K, H, F = 16, 8, 2816, 704
    pool = synth.expert_pool(E, H, F, 35)
    layer = gpu.MoeLayer(pool, E, H, F, K)
    layer.tolerance_class = tolerance_class
    lib = gpu.load()
    stream = lib.salt_mi355_stream()
    scale = np.ones(E, np.float32)
    layer.step(synth.router_logits(E, 1000), scale, synth.activations(H, 1, 1001)[0])     # first use outside the capture
    gpu.check(lib.salt_mi355_graph_begin(stream), "graph_begin")
    for _ in range(4):
        gpu.check(layer.enqueue(stream), "captured step")
    graph = lib.salt_mi355_graph_end(stream)
    assert graph, lib.salt_mi355_last_error().decode()
    for it in range(4):
        logits, x = synth.router_logits(E, 1010 + it), synth.activations(H, 1, 1020 + it)[0]
        if it == 2:
            logits = logits.copy(); logits[5] = np.nan                # a rejected step inside a replay
        want = layer.step(logits, scale, x)                            # eager, also the work between replays
        layer.out.upload(np.full(H, 7.0, np.float32))
        gpu.check(lib.salt_mi355_graph_launch(graph, stream), "graph_launch")
        gpu.check(lib.salt_mi355_stream_sync(stream), "sync")
        status, out = int(layer.ws.to_host(np.int32, 1)[0]), layer.out.to_host(np.float32)
        assert status == want[0] == (-1 if it == 2 else 0)
        if it == 2:
            assert (out == 7.0).all()
        else:
            assert np.array_equal(bits(out), bits(want[4])), it
            assert np.array_equal(bits(layer.eo.to_host(np.float32).reshape(K, H)), bits(want[3]))
    assert lib.salt_mi355_graph_destroy(graph) == 0


def test_moe_decode_step_behind_a_pool_file_header(gpu, oracle):
    """Expert 0 starts 24 bytes into the allocation, as in the engine's pool file (three 64-bit header words): every
    tensor of every expert is then 8 bytes past a multiple of 16."""
    print("moe step, pool behind a 24-byte header", flush=True)
    E, K, H, F = 16, 8, 2816, 704
    pool = synth.expert_pool(E, H, F, 33)
    layer = gpu.MoeLayer(pool, E, H, F, K, header_bytes=24)
    g = ExpertGeometry(H, F)
    scale = synth.rng(3).uniform(0.5, 2.0, E).astype(np.float32)
    logits = synth.router_logits(E, 71); x = synth.activations(H, 1, 72)[0]
    st, sel, w, eo, y = layer.step(logits, scale, x)
    osel = np.zeros(K, np.int32); ow = np.zeros(K, np.float32)
    oeo = np.zeros((K, H), np.float32); oy = np.zeros(H, np.float32)
    assert oracle.orc_moe_decode_step(C.byref(g), ptr(pool), E, K, ptr(logits), ptr(scale), ptr(x), ptr(osel), ptr(ow),
                                      ptr(oeo), ptr(oy), host_threads()) == 0
    assert st == 0 and np.array_equal(sel, osel) and np.array_equal(bits(w), bits(ow))
    assert np.array_equal(bits(eo), bits(oeo)) and np.array_equal(bits(y), bits(oy))


@pytest.mark.parametrize("E,K,H,F,why", [
    (520, 4, 128, 64, "more experts than the fused prologue holds: router, gate/up, activate, down, reduce as five launches"),
    (16, 16, 2816, 2048, "more than two tiles per compute unit: eight waves per tile in both fused launches"),
    (24, 5, 192, 4160, "d_ff beyond the LDS activation buffer of the fused down launch: five launches"),
    (16, 4, 4160, 128, "65 row tiles in the down launch, two tiles in each gate and up projection"),
    (580, 1, 384, 320, "five launches with a single selected expert: the down launch's table holds one job"),
])
def test_moe_decode_step_other_launch_shapes(gpu, oracle, E, K, H, F, why):
    print(f"moe step E={E} K={K} H={H} F={F}: {why}", flush=True)
    pool = synth.expert_pool(E, H, F, E + K)
    layer = gpu.MoeLayer(pool, E, H, F, K)
    g = ExpertGeometry(H, F)
    scale = synth.rng(2).uniform(0.5, 2.0, E).astype(np.float32)
    logits = synth.router_logits(E, 40 + E); x = synth.activations(H, 1, 41 + E)[0]
    st, sel, w, eo, y = layer.step(logits, scale, x)
    osel = np.zeros(K, np.int32); ow = np.zeros(K, np.float32)
    oeo = np.zeros((K, H), np.float32); oy = np.zeros(H, np.float32)
    assert oracle.orc_moe_decode_step(C.byref(g), ptr(pool), E, K, ptr(logits), ptr(scale), ptr(x), ptr(osel),
                                      ptr(ow), ptr(oeo), ptr(oy), host_threads()) == 0
    assert st == 0 and np.array_equal(sel, osel) and np.array_equal(bits(w), bits(ow))
    assert np.array_equal(bits(eo), bits(oeo)) and np.array_equal(bits(y), bits(oy))
    logits[E - 1] = np.nan
    assert layer.step(logits, scale, x)[0] == -1
