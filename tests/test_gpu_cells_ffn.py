"""The fp32 cells around the MoE step (norms, router input, residual post-norm, parallel combine, softcap, top-k) and
the whole feed-forward block of a decoder layer on the MI355X through the C ABI, bit-for-bit against the CPU checker."""
import ctypes as C

import numpy as np
import pytest

from golden import cases
from oracle_lib import bits, ffn_layer_struct, host_threads, ptr

pytestmark = pytest.mark.gpu
synth = cases.synth
f32 = np.float32


@pytest.fixture(scope="module")
def gpu(pkg):
    pkg.lib.init()
    return pkg.lib


def vectors(n, seed):
    g = synth.rng(seed)
    mk = lambda s: (g.standard_normal(n) * s).astype(f32)
    return {"x": mk(3), "w": mk(1), "w2": mk(1), "w3": mk(1), "res": mk(2), "dense": mk(5), "routed": mk(0.01),
            "out": np.full(n, np.nan, f32), "scratch": np.zeros(2 * n, f32)}


@pytest.mark.parametrize("n", [2816, 64, 1, 4097, 9000])
def test_each_cell_kind_matches_the_checker(gpu, oracle, n):
    print("cells n", n, flush=True)
    v = vectors(n, n)
    eps = f32(1e-6)
    want = np.zeros(n, f32)
    for aux in (0, 1):
        st, got = gpu.run_cells([(gpu.CELL_RMSNORM, ["x", "w", "out"], n, aux, eps, 0.0)], v)
        assert oracle.orc_rmsnorm(ptr(want), ptr(v["x"]), ptr(v["w"]), n, eps, aux) == 0
        assert st == 0 and np.array_equal(bits(got["out"]), bits(want)), aux
    for scalar in (0.0, float(f32(1.0) / f32(oracle.orc_sqrtf(f32(n))))):
        st, got = gpu.run_cells([(gpu.CELL_ROUTER_INPUT, ["x", "w", "out"], n, 0, eps, scalar)], v)
        assert oracle.orc_router_input(ptr(want), ptr(v["x"]), ptr(v["w"]), n, eps) == 0
        assert st == 0 and np.array_equal(bits(got["out"]), bits(want)), scalar
    st, got = gpu.run_cells([(gpu.CELL_RESIDUAL_POSTNORM, ["res", "x", "w", "out"], n, 0, eps, 0.0)], v)
    assert oracle.orc_residual_postnorm(ptr(want), ptr(v["res"]), ptr(v["x"]), ptr(v["w"]), n, eps) == 0
    assert st == 0 and np.array_equal(bits(got["out"]), bits(want)) and np.array_equal(bits(got["x"]), bits(v["x"]))
    st, got = gpu.run_cells([(gpu.CELL_PARALLEL_COMBINE, ["res", "dense", "routed", "w", "w2", "w3", "scratch", "out"], n, 0,
                              eps, 0.37)], v)
    assert oracle.orc_parallel_ffn_combine(ptr(want), ptr(v["res"]), ptr(v["dense"]), ptr(v["routed"]), ptr(v["w"]),
                                           ptr(v["w2"]), ptr(v["w3"]), f32(0.37), n, eps) == 0
    assert st == 0 and np.array_equal(bits(got["out"]), bits(want))
    logits = {"l": (v["dense"] * 8).astype(f32)}
    st, got = gpu.run_cells([(gpu.CELL_SOFTCAP, ["l"], n, 0, 0.0, 30.0)], logits)
    capped = logits["l"].copy()
    assert oracle.orc_softcap(ptr(capped), n, f32(30.0)) == 0
    assert st == 0 and np.array_equal(bits(got["l"]), bits(capped))


def test_cells_run_in_order_alias_and_reject(gpu, oracle):
    print("cells sequence", flush=True)
    n = 2816
    v = vectors(n, 7)
    eps = f32(1e-6)
    # in-place norm, then a residual post-norm that reads it, then the router input of that: three dependent cells
    seq = [(gpu.CELL_RMSNORM, ["x", "w", "x"], n, 1, eps, 0.0),
           (gpu.CELL_RESIDUAL_POSTNORM, ["res", "x", "w2", "out"], n, 0, eps, 0.0),
           (gpu.CELL_ROUTER_INPUT, ["out", "w3", "dense"], n, 0, eps, 0.0)]
    st, got = gpu.run_cells(seq, v)
    a = v["x"].copy(); b = np.zeros(n, f32); c = np.zeros(n, f32)
    assert oracle.orc_rmsnorm(ptr(a), ptr(a), ptr(v["w"]), n, eps, 1) == 0
    assert oracle.orc_residual_postnorm(ptr(b), ptr(v["res"]), ptr(a), ptr(v["w2"]), n, eps) == 0
    assert oracle.orc_router_input(ptr(c), ptr(b), ptr(v["w3"]), n, eps) == 0
    assert st == 0 and np.array_equal(bits(got["x"]), bits(a)) and np.array_equal(bits(got["out"]), bits(b))
    assert np.array_equal(bits(got["dense"]), bits(c))
    # a non-finite element: that cell and every later one publish nothing
    bad = dict(v); bad["res"] = v["res"].copy(); bad["res"][99] = np.inf
    st, got = gpu.run_cells(seq, bad)
    assert st == -1 and np.array_equal(bits(got["x"]), bits(a))
    assert np.isnan(got["out"]).all() and np.array_equal(bits(got["dense"]), bits(v["dense"]))
    for kind, names, field in [(gpu.CELL_RMSNORM, ["x", "w", "out"], "x"), (gpu.CELL_RMSNORM, ["x", "w", "out"], "w"),
                               (gpu.CELL_ROUTER_INPUT, ["x", "w", "out"], "w"),
                               (gpu.CELL_PARALLEL_COMBINE, ["res", "dense", "routed", "w", "w2", "w3", "scratch", "out"], "routed"),
                               (gpu.CELL_PARALLEL_COMBINE, ["res", "dense", "routed", "w", "w2", "w3", "scratch", "out"], "w3")]:
        bad = dict(v); bad[field] = v[field].copy(); bad[field][n - 1] = np.nan
        st, got = gpu.run_cells([(kind, names, n, 1, eps, 1.0)], bad)
        assert st == -1 and np.isnan(got["out"]).all(), (kind, field)
    st, got = gpu.run_cells([(gpu.CELL_RMSNORM, ["x", "w", "out"], n, 0, f32(-1.0), 0.0)], v)
    assert st == -1
    big = {"l": np.array([1.0, np.inf, 3.0, 4.0], f32)}
    st, got = gpu.run_cells([(gpu.CELL_SOFTCAP, ["l"], 4, 0, 0.0, 30.0)], big)
    assert st == -1 and np.array_equal(bits(got["l"]), bits(big["l"]))
    # the serial sum of squares: 2^24 then ones stays 2^24
    x = np.ones(4096, f32); x[0] = 4096.0
    st, got = gpu.run_cells([(gpu.CELL_RMSNORM, ["x", "x", "out"], 4096, 0, 0.0, 0.0)], {"x": x, "out": np.zeros(4096, f32)})
    want = np.zeros(4096, f32)
    assert oracle.orc_rmsnorm(ptr(want), ptr(x), None, 4096, 0.0, 0) == 0
    assert st == 0 and np.array_equal(bits(got["out"]), bits(want))
    # refused before anything is enqueued
    lib = gpu.load()
    buf = gpu.DeviceBuffer(4096, fill=0)
    cell = gpu.Cell(9, (C.c_void_p * 8)(buf.ptr, buf.ptr, buf.ptr), 4, 0, 0.0, 0.0)
    assert lib.salt_mi355_cells_dev(C.byref(cell), 1, buf.ptr, None) == -1
    cell = gpu.Cell(gpu.CELL_RMSNORM, (C.c_void_p * 8)(buf.ptr, None, buf.ptr), 4, 1, 0.0, 0.0)
    assert lib.salt_mi355_cells_dev(C.byref(cell), 1, buf.ptr, None) == -1
    cell = gpu.Cell(gpu.CELL_SOFTCAP, (C.c_void_p * 8)(buf.ptr), 4, 0, 0.0, -1.0)
    assert lib.salt_mi355_cells_dev(C.byref(cell), 1, buf.ptr, None) == -1


def test_topk_cell_sorts_by_expert(gpu, oracle):
    print("cells topk", flush=True)
    E, K = 128, 8
    logits = synth.router_logits(E, 5); scale = synth.rng(6).uniform(0.5, 2.0, E).astype(f32)
    arrays = {"logits": logits, "scale": scale, "sel": np.full(K, -7, np.int32), "w": np.zeros(K, f32)}
    st, got = gpu.run_cells([(gpu.CELL_TOPK, ["logits", "scale", "sel", "w"], E, K, 0.0, 0.0)], arrays)
    sel = np.zeros(K, np.int32); w = np.zeros(K, f32)
    assert oracle.orc_router_topk(ptr(logits), ptr(scale), E, K, ptr(sel), ptr(w)) == 0
    oracle.orc_sort_selection(ptr(sel), ptr(w), K)
    assert st == 0 and np.array_equal(got["sel"], sel) and np.array_equal(bits(got["w"]), bits(w))
    arrays["logits"] = logits.copy(); arrays["logits"][3] = np.nan
    st, got = gpu.run_cells([(gpu.CELL_TOPK, ["logits", "scale", "sel", "w"], E, K, 0.0, 0.0)], arrays)
    assert st == -1 and (got["sel"] == -7).all()


@pytest.mark.parametrize("H,D,F,E,K,seed", [(256, 192, 128, 16, 4, 1), (2816, 2112, 704, 16, 8, 2), (2816, 2112, 704, 128, 8, 3)])
def test_ffn_block_matches_the_checker(gpu, oracle, H, D, F, E, K, seed):
    print("ffn block", H, D, F, E, K, flush=True)
    w = synth.ffn_layer(H, D, F, E, K, seed)
    block = gpu.FfnBlock(w)
    L = ffn_layer_struct(w)
    for it in range(2):
        residual = (synth.activations(H, 1, 90 + seed + it)[0] * 3).astype(f32)
        st, sel, wt, out = block.step(residual)
        want = np.zeros(H, f32); osel = np.zeros(K, np.int32); owt = np.zeros(K, f32)
        assert oracle.orc_ffn_block(C.byref(L), ptr(residual), ptr(want), ptr(osel), ptr(owt), host_threads()) == 0
        assert st == 0 and np.array_equal(sel, osel) and np.array_equal(bits(wt), bits(owt))
        assert np.array_equal(bits(out), bits(want))
    # a non-finite residual: status -1, the previous output stays
    residual[5] = np.inf
    st, _, _, out2 = block.step(residual)
    assert st == -1 and np.array_equal(bits(out2), bits(out))
    # and the block recovers on the next call
    residual[5] = 0.25
    st, _, _, out3 = block.step(residual)
    assert oracle.orc_ffn_block(C.byref(L), ptr(residual), ptr(want), None, None, host_threads()) == 0
    assert st == 0 and np.array_equal(bits(out3), bits(want))


def test_ffn_block_argument_errors(gpu):
    w = synth.ffn_layer(256, 192, 128, 4, 2, 9)
    block = gpu.FfnBlock(w)
    lib = gpu.load()
    d = block.desc
    args = lambda desc, res, out, ws: lib.salt_mi355_ffn_block_dev(C.byref(desc), res, out, block.sel.ptr, block.w.ptr,
                                                                   block.status.ptr, ws, None)
    assert args(d, block.residual.ptr, block.residual.ptr, block.ws.ptr) == -1          # out aliases the residual
    assert args(d, block.residual.ptr, block.out.ptr, block.ws.ptr + 4) == -1           # misaligned workspace
    bad = type(d).from_buffer_copy(d); bad.hidden = 250
    assert args(bad, block.residual.ptr, block.out.ptr, block.ws.ptr) == -1 and lib.salt_mi355_ffn_block_workspace_bytes(C.byref(bad)) == 0
    bad = type(d).from_buffer_copy(d); bad.topk = 5
    assert args(bad, block.residual.ptr, block.out.ptr, block.ws.ptr) == -1


def test_block_replayed_as_a_graph(gpu, oracle):
    """The feed-forward block (two streams forked and joined by events, kernels only: no memset node; the MoE decode
    step is part of it) captured once and replayed with fresh inputs; every replay is compared with the checker, with
    eager calls and synchronisations in between."""
    print("graph replay", flush=True)
    H, D, F, E, K = 2816, 2112, 704, 16, 8
    w = synth.ffn_layer(H, D, F, E, K, 5)
    block = gpu.FfnBlock(w)
    L = ffn_layer_struct(w)
    lib = gpu.load()
    stream = lib.salt_mi355_stream()
    block.residual.upload((synth.activations(H, 1, 300)[0] * 3).astype(f32))
    gpu.check(block.enqueue(stream), "eager warm-up")              # first use outside the capture
    gpu.check(lib.salt_mi355_stream_sync(stream), "sync")
    gpu.check(lib.salt_mi355_graph_begin(stream), "graph_begin")
    gpu.check(block.enqueue(stream), "captured block")
    graph = lib.salt_mi355_graph_end(stream)
    assert graph, lib.salt_mi355_last_error().decode()
    want = np.zeros(H, f32); osel = np.zeros(K, np.int32); owt = np.zeros(K, f32)
    for it in range(4):
        residual = (synth.activations(H, 1, 301 + it)[0] * 3).astype(f32)
        if it == 2:
            residual[9] = np.nan                                      # a rejected input inside a replay
        block.residual.upload(residual)
        block.out.upload(np.full(H, 7.0, f32))
        gpu.check(lib.salt_mi355_graph_launch(graph, stream), "graph_launch")
        gpu.check(lib.salt_mi355_stream_sync(stream), "sync")
        status, out = int(block.status.to_host(np.int32)[0]), block.out.to_host(f32)
        if it == 2:
            assert status == -1 and (out == 7.0).all()
        else:
            assert oracle.orc_ffn_block(C.byref(L), ptr(residual), ptr(want), ptr(osel), ptr(owt), host_threads()) == 0
            assert status == 0 and np.array_equal(bits(out), bits(want)), it
            assert np.array_equal(block.sel.to_host(np.int32), osel)
        # an eager call between replays
        st, _, _, eager = block.step((synth.activations(H, 1, 400 + it)[0] * 3).astype(f32))
        assert st == 0
    assert lib.salt_mi355_graph_destroy(graph) == 0
