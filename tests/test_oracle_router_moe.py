"""Pins the transcendental, router and routed-expert parts of the CPU checker.

The reference tree holds no vectors for these (its own tests for them are not
shipped), so they are pinned by what the mathematics fixes, by the reference's
own sources when compiled, and by tests/golden fixtures made from those."""
import ctypes as C
import math

import numpy as np
import pytest

from oracle_lib import ExpertGeometry, bits, ptr
from __graft_entry__ import load_package

synth = load_package().synth


def sample_points():
    g = synth.rng(41)
    return np.concatenate([
        g.uniform(-90, 90, 4000), g.uniform(-1, 1, 2000), g.standard_normal(2000) * 4,
        [0.0, -0.0, 88.722839, 88.72284, -87.336548, -87.33655, 1e-8, -1e-8, 10.0, -10.0, 9.999999,
         0.34657359, -0.34657359, 0.6931472, np.inf, -np.inf]]).astype(np.float32)


def test_expf_close_to_libm_and_edges(oracle):
    for v in sample_points():
        got = oracle.orc_expf(float(v))
        if v > 88.722839:
            assert got == np.float32(3.402823466e+38)
        elif v < -87.336548:
            assert got == 0.0
        else:
            want = math.exp(float(v))
            if want > 3.4028234e38:      # at the upper guard itself ldexpf overflows
                assert got == np.inf
                continue
            assert abs(got - want) <= 4e-7 * want, float(v)
    assert np.isnan(oracle.orc_expf(float("nan")))
    assert oracle.orc_expf(0.0) == 1.0


def test_tanhf_and_gelu_close_to_closed_forms(oracle):
    k = 0.7978845608028654
    for v in sample_points():
        v = float(v)
        t = oracle.orc_tanhf(v)
        assert abs(t - math.tanh(v)) <= 3e-7, v
        assert oracle.orc_tanhf(-v) == -t or v == 0.0
        if abs(v) < 50:
            want = 0.5 * v * (1.0 + math.tanh(k * (v + 0.044715 * v ** 3)))
            assert abs(oracle.orc_gelu_tanh(v) - want) <= 1e-6 * max(1.0, abs(want)), v
    assert oracle.orc_tanhf(10.0) == 1.0 and oracle.orc_tanhf(-10.0) == -1.0
    assert oracle.orc_gelu_tanh(0.0) == 0.0


def run_topk(lib_fn, logits, scale, k):
    sel = np.full(k, -7, np.int32); w = np.full(k, -7, np.float32)
    rc = lib_fn(ptr(logits), ptr(scale), len(logits), k, ptr(sel), ptr(w))
    return rc, sel, w


@pytest.mark.parametrize("E,k,seed", [(8, 2, 1), (16, 4, 2), (128, 8, 3), (128, 8, 4), (5, 5, 5), (7, 1, 6)])
def test_router_topk_order_and_weights(oracle, E, k, seed):
    g = synth.rng(seed)
    logits = g.standard_normal(E).astype(np.float32)
    if seed % 2 == 0:           # force ties: quantise the logits coarsely
        logits = (np.round(logits * 2) / 2).astype(np.float32)
    scale = g.uniform(0.5, 2.0, E).astype(np.float32)
    rc, sel, w = run_topk(oracle.orc_router_topk, logits, scale, k)
    assert rc == 0
    # brute force: descending logit, lower index first on ties
    order = sorted(range(E), key=lambda e: (-float(logits[e]), e))[:k]
    assert list(sel) == order
    ex = np.exp(logits.astype(np.float64) - float(logits.max()))
    p = ex[order] / ex.sum()
    want = p / p.sum() * scale[order]
    assert np.allclose(w, want, rtol=2e-6, atol=0)
    # with unit scales the weights sum to one
    rc, _, w1 = run_topk(oracle.orc_router_topk, logits, np.ones(E, np.float32), k)
    assert rc == 0 and abs(float(w1.astype(np.float64).sum()) - 1.0) < 1e-6


def test_router_topk_rejects_and_leaves_outputs(oracle):
    logits = np.zeros(8, np.float32); scale = np.ones(8, np.float32)
    for bad in (np.inf, np.nan):
        l2 = logits.copy(); l2[3] = bad
        rc, sel, w = run_topk(oracle.orc_router_topk, l2, scale, 2)
        assert rc == -1 and (sel == -7).all() and (w == -7).all()
    s2 = scale.copy(); s2[0] = np.nan
    assert run_topk(oracle.orc_router_topk, logits, s2, 2)[0] == -1
    assert run_topk(oracle.orc_router_topk, logits, scale, 9)[0] == -1
    sel = np.zeros(2, np.int32)
    assert oracle.orc_router_topk(ptr(logits), ptr(scale), 8, 2, ptr(sel), ptr(logits)) == -1  # aliasing
    # all-equal logits: the first k experts, equal weights
    rc, sel, w = run_topk(oracle.orc_router_topk, logits, scale, 3)
    assert rc == 0 and list(sel) == [0, 1, 2] and np.allclose(w, 1 / 3, rtol=1e-6)


def test_sort_selection(oracle):
    sel = np.array([9, 2, 7, 0, 5], np.int32); w = np.array([.9, .2, .7, .0, .5], np.float32)
    oracle.orc_sort_selection(ptr(sel), ptr(w), 5)
    assert list(sel) == [0, 2, 5, 7, 9] and np.array_equal(w, np.array([.0, .2, .5, .7, .9], np.float32))


def test_mix64_is_splitmix64(oracle):
    # first outputs of splitmix64 seeded with 0 (Vigna's reference values): each
    # output is mix64 of the running state, which advances by the golden gamma
    gamma = 0x9E3779B97F4A7C15
    want = [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    for i, value in enumerate(want):
        assert oracle.orc_mix64((gamma * i) & (2 ** 64 - 1)) == value


def py_mix64(x):
    M = 2 ** 64 - 1
    x = (x + 0x9E3779B97F4A7C15) & M
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & M
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & M
    return x ^ (x >> 31)


@pytest.mark.parametrize("locality", [0.0, 0.75])
def test_router_fixture_against_python_restatement(oracle, locality):
    E, K, state, layer = 128, 8, 0x1234567890ABCDEF, 17
    M = 2 ** 64 - 1
    h3 = lambda a, b, c: py_mix64(a ^ py_mix64((b * 0x100000001B3 + c) & M))
    sc, ch = [], []
    for e in range(E):
        acc = (h3(state, layer, e) & 0xFFFFFF) / 16777216.0
        bias = (h3(state ^ 0xB1A5, layer, e) & 0xFFFFFF) / 16777216.0
        sel = acc + (bias - 0.5) * 0.1
        if locality > 0:
            sel = acc * (1.0 + locality * (1.0 / (1.0 + (e % 64))))
        sc.append(np.float32(acc)); ch.append(np.float32(sel))
    order = sorted(range(E), key=lambda e: (-float(ch[e]), e))[:K]
    idx = np.zeros(K, np.int32); w = np.zeros(K, np.float32)
    assert oracle.orc_router_fixture(ptr(idx), ptr(w), E, K, state, layer, locality) == 0
    assert list(idx) == order
    assert np.array_equal(bits(w), bits(np.array([sc[e] for e in order], np.float32)))


def small_geometry():
    return ExpertGeometry(128, 64)


def test_expert_ffn_is_the_composition(oracle):
    g = small_geometry()
    H, F = g.hidden, g.routed
    pool = synth.expert_pool(2, H, F, 3)
    assert oracle.orc_expert_slot_bytes(C.byref(g)) == synth.expert_slot_bytes(H, F)
    x = synth.activations(H, 1, 4)[0]
    gate = np.zeros(F, np.float32); up = np.zeros(F, np.float32); out = np.zeros(H, np.float32)
    slot = pool[synth.expert_slot_bytes(H, F):]
    assert oracle.orc_expert_ffn(C.byref(g), ptr(slot), ptr(x), ptr(gate), ptr(up), ptr(out)) == 0
    gv = synth.expert_views(pool, 1, 0, H, F); uv = synth.expert_views(pool, 1, 1, H, F)
    dv = synth.expert_views(pool, 1, 2, H, F)
    g1 = np.zeros(F, np.float32); u1 = np.zeros(F, np.float32); o1 = np.zeros(H, np.float32)
    oracle.orc_q4_matvec(ptr(gv[0]), ptr(gv[1]), ptr(gv[2]), F, H, ptr(x), ptr(g1))
    oracle.orc_q4_matvec(ptr(uv[0]), ptr(uv[1]), ptr(uv[2]), F, H, ptr(x), ptr(u1))
    h = np.array([np.float32(oracle.orc_gelu_tanh(float(a))) * b for a, b in zip(g1, u1)], np.float32)
    oracle.orc_q4_matvec(ptr(dv[0]), ptr(dv[1]), ptr(dv[2]), H, F, ptr(h), ptr(o1))
    assert np.array_equal(bits(gate), bits(h)) and np.array_equal(bits(up), bits(u1))
    assert np.array_equal(bits(out), bits(o1))


def test_decode_step_reduces_in_ascending_expert_order(oracle):
    g = small_geometry()
    H, F, E, K = g.hidden, g.routed, 8, 3
    pool = synth.expert_pool(E, H, F, 5)
    logits = synth.router_logits(E, 6); scale = np.ones(E, np.float32)
    x = synth.activations(H, 1, 7)[0]
    sel = np.zeros(K, np.int32); w = np.zeros(K, np.float32)
    eo = np.zeros((K, H), np.float32); out = np.zeros(H, np.float32)
    assert oracle.orc_moe_decode_step(C.byref(g), ptr(pool), E, K, ptr(logits), ptr(scale), ptr(x),
                                      ptr(sel), ptr(w), ptr(eo), ptr(out), 2) == 0
    assert list(sel) == sorted(sel) and set(sel) == set(np.argsort(-logits, kind="stable")[:K])
    acc = np.zeros(H, np.float32)
    slot = synth.expert_slot_bytes(H, F)
    for i in range(K):
        gate = np.zeros(F, np.float32); up = np.zeros(F, np.float32); o = np.zeros(H, np.float32)
        oracle.orc_expert_ffn(C.byref(g), ptr(pool[sel[i] * slot:]), ptr(x), ptr(gate), ptr(up), ptr(o))
        assert np.array_equal(bits(o), bits(eo[i]))
        acc = (acc + (o * w[i]).astype(np.float32)).astype(np.float32)
    assert np.array_equal(bits(out), bits(acc))


def test_group_equals_per_token_steps_and_validates(oracle):
    g = small_geometry()
    H, F, E, K, T = g.hidden, g.routed, 8, 2, 9
    pool = synth.expert_pool(E, H, F, 8)
    sel, w = synth.zipf_selection(T, E, K, 1.1, 9)
    xs = synth.activations(H, T, 10)
    out = np.zeros((T, H), np.float32); rows = np.zeros(E, np.int32)
    assert oracle.orc_moe_group(C.byref(g), ptr(pool), E, K, T, ptr(sel), ptr(w), ptr(xs), ptr(out), ptr(rows), 3) == 0
    assert rows.sum() == T * K and np.array_equal(rows, np.bincount(sel.ravel(), minlength=E))
    slot = synth.expert_slot_bytes(H, F)
    for t in range(T):
        acc = np.zeros(H, np.float32)
        for k in range(K):
            gate = np.zeros(F, np.float32); up = np.zeros(F, np.float32); o = np.zeros(H, np.float32)
            oracle.orc_expert_ffn(C.byref(g), ptr(pool[sel[t, k] * slot:]), ptr(xs[t]), ptr(gate), ptr(up), ptr(o))
            acc = (acc + (o * w[t, k]).astype(np.float32)).astype(np.float32)
        assert np.array_equal(bits(out[t]), bits(acc))
    bad = sel.copy(); bad[4, 1] = bad[4, 0]
    assert oracle.orc_moe_group(C.byref(g), ptr(pool), E, K, T, ptr(bad), ptr(w), ptr(xs), ptr(out), None, 1) == -1
    bad = sel.copy(); bad[0, 0] = E
    assert oracle.orc_moe_group(C.byref(g), ptr(pool), E, K, T, ptr(bad), ptr(w), ptr(xs), ptr(out), None, 1) == -1
    wb = w.copy(); wb[2, 1] = np.nan
    assert oracle.orc_moe_group(C.byref(g), ptr(pool), E, K, T, ptr(sel), ptr(wb), ptr(xs), ptr(out), None, 1) == -1


# ---- against the reference's own sources, when they have been compiled ----

def test_transcendentals_equal_compiled_reference(oracle, reference):
    pts = np.concatenate([sample_points(), synth.rng(43).uniform(-12, 12, 20000).astype(np.float32)])
    for v in pts:
        v = float(v)
        for a, b in ((oracle.orc_expf, reference.salt_expf), (oracle.orc_tanhf, reference.salt_tanhf),
                     (oracle.orc_gelu_tanh, reference.salt_gemma4_gelu_tanh)):
            x, y = np.float32(a(v)), np.float32(b(v))
            assert bits(x) == bits(y) or (np.isnan(x) and np.isnan(y)), v


@pytest.mark.parametrize("seed", range(12))
def test_router_topk_equals_compiled_reference(oracle, reference, seed):
    g = synth.rng(100 + seed)
    E, k = (128, 8) if seed % 3 else (64, 6)
    logits = g.standard_normal(E).astype(np.float32)
    if seed % 2:
        logits = (np.round(logits * 3) / 3).astype(np.float32)
    scale = g.uniform(0.25, 4.0, E).astype(np.float32)
    a = run_topk(oracle.orc_router_topk, logits, scale, k)
    b = run_topk(reference.salt_gemma4_router_topk, logits, scale, k)
    assert a[0] == b[0] == 0 and np.array_equal(a[1], b[1]) and np.array_equal(bits(a[2]), bits(b[2]))


def test_mix64_equals_compiled_reference(oracle, reference):
    for v in [0, 1, 2 ** 64 - 1, 0xDEADBEEF, 0x9E3779B97F4A7C15]:
        assert oracle.orc_mix64(v) == reference.salt_mix64(v)


def test_decode_step_and_group_equal_the_reference_driven_through_its_public_functions(oracle, reference):
    """oracle/ref_moe_driver.c calls the reference's own router, matvecs, gelu and grouped executor in the order of
    its (static) MoE step; the checker's step and group must give the same bits."""
    if not hasattr(reference, "refdrv_moe_decode_step"):
        pytest.skip("the reference library was built without the driver")
    E, K, H, F = 16, 4, 256, 128
    pool = synth.expert_pool(E, H, F, 71)
    stride = synth.expert_slot_bytes(H, F)
    g = ExpertGeometry(H, F)
    logits, scale = synth.router_logits(E, 72), (1.0 + 0.1 * synth.router_logits(E, 73)).astype(np.float32)
    x = synth.activations(H, 1, 74)[0]
    sel, w, eo, y = np.zeros(K, np.int32), np.zeros(K, np.float32), np.zeros((K, H), np.float32), np.zeros(H, np.float32)
    assert oracle.orc_moe_decode_step(C.byref(g), ptr(pool), E, K, ptr(logits), ptr(scale), ptr(x), ptr(sel), ptr(w),
                                      ptr(eo), ptr(y), 2) == 0
    rsel, rw, reo, ry = np.zeros(K, np.int32), np.zeros(K, np.float32), np.zeros((K, H), np.float32), np.zeros(H, np.float32)
    scratch = np.zeros(K * (2 * F + H), np.float32)
    for threads in (1, 3):
        assert reference.refdrv_moe_decode_step(ptr(pool), stride, E, K, H, F, ptr(logits), ptr(scale), ptr(x), ptr(rsel),
                                                ptr(rw), ptr(reo), ptr(ry), ptr(scratch), threads) == 0
        assert np.array_equal(rsel, sel) and np.array_equal(bits(rw), bits(w))
        assert np.array_equal(bits(reo), bits(eo)) and np.array_equal(bits(ry), bits(y))
    T = 9
    gsel, gw = synth.zipf_selection(T, E, K, 1.1, 75)
    xs = synth.activations(H, T, 76)
    want, got = np.zeros((T, H), np.float32), np.zeros((T, H), np.float32)
    assert oracle.orc_moe_group(C.byref(g), ptr(pool), E, K, T, ptr(gsel), ptr(gw), ptr(xs), ptr(want), None, 2) == 0
    gscratch = np.zeros(T * (2 * F + 2 * H + K * H), np.float32)
    assert reference.refdrv_moe_group(ptr(pool), stride, E, K, H, F, T, ptr(gsel), ptr(gw), ptr(xs), ptr(got),
                                      ptr(gscratch)) == 0
    assert np.array_equal(bits(got), bits(want))
