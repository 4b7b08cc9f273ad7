"""Grouped prefill MoE on the device.

Index work (rows per expert, the order of the grouped rows) is bit-exact
against the reference's grouping (src/moe_group.c:138-184) as recorded in the
golden fixtures and as recomputed here.  Values run on the matrix-core matmul
and carry a stated tolerance against the bit-exact CPU checker:

    |error[token][d]| <= 2^-18 * M[token][d] + 1e-6,
    M[token][d] = sum over the token's experts k of |w_k| * sum_f |Wd_k[d][f] * h_k[f]|

per output, where h_k = gelu_tanh(gate_k) * up_k is the expert's activation and Wd_k its dequantised down projection
(the sum of the magnitudes of the terms that make up the output; test_against_cpu_checker computes it in float64).
At the full BASELINE geometry the fixtures hold outputs only; there the bound is per token,
2^-18 * max_d |y[token][d]| + 1e-6."""
import ctypes as C

import numpy as np
import pytest

from golden import cases
from moe_bounds import group_term_magnitudes as term_magnitudes
from oracle_lib import ExpertGeometry, host_threads, ptr

pytestmark = pytest.mark.gpu
synth = cases.synth


def expected_grouping(sel, E):
    """(rows per expert, pair index of each grouped row): ascending expert, then token, then rank."""
    flat = sel.ravel()
    order = np.argsort(flat, kind="stable").astype(np.int32)
    return np.bincount(flat, minlength=E).astype(np.int32), order


def check_values(got, want, magnitudes=None):
    scale = np.abs(want).max(axis=1, keepdims=True).astype(np.float64) if magnitudes is None else magnitudes
    bound = 2.0 ** -18 * scale + 1e-6
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    ratio = float((err / bound).max())
    print("max err / bound", ratio, flush=True)
    assert np.isfinite(got).all() and ratio <= 1.0, ratio


@pytest.mark.parametrize("case", cases.GROUP_CASES, ids=lambda c: c[0])
def test_golden_group_cases(pkg, case):
    name, T, E, K, H, F, _, pseed, sseed = case
    print("prefill golden", name, flush=True)
    fx = cases.load("moe_group.npz")
    pool, sel, w, xs = cases.group_case_inputs(T, E, K, H, F, pseed, sseed)
    assert cases.pool_digest(pool, xs) == str(fx[name + ".digest"])
    layer = pkg.lib.MoePrefill(pool, E, H, F, K, T)
    status, ys, rows, pairs = layer.run(sel, w, xs)
    assert status == 0
    used = np.nonzero(rows)[0]
    assert np.array_equal(used, fx[name + ".run_experts"]) and np.array_equal(rows[used], fx[name + ".run_rows"])
    want_rows, want_pairs = expected_grouping(sel, E)
    assert np.array_equal(rows, want_rows) and np.array_equal(pairs, want_pairs)
    check_values(ys, fx[name + ".y_bits"].view(np.float32).reshape(T, H))


@pytest.mark.parametrize("T,E,K,H,F", [(300, 16, 4, 256, 128), (1, 8, 3, 128, 64), (130, 5, 5, 192, 320),
                                       (65, 128, 8, 128, 128)])
def test_against_cpu_checker(pkg, oracle, T, E, K, H, F):
    print(f"prefill T={T} E={E} K={K} H={H} F={F}", flush=True)
    pool = synth.expert_pool(E, H, F, T + E)
    sel, w = synth.zipf_selection(T, E, K, 1.1, 31 + T)
    xs = synth.activations(H, T, 32 + T)
    g = ExpertGeometry(H, F)
    want = np.zeros((T, H), np.float32)
    assert oracle.orc_moe_group(C.byref(g), ptr(pool), E, K, T, ptr(sel), ptr(w), ptr(xs), ptr(want), None,
                                host_threads()) == 0
    layer = pkg.lib.MoePrefill(pool, E, H, F, K, T + 7)       # workspace larger than the call
    status, ys, rows, pairs = layer.run(sel, w, xs)
    assert status == 0
    want_rows, want_pairs = expected_grouping(sel, E)
    assert np.array_equal(rows, want_rows) and np.array_equal(pairs, want_pairs)
    check_values(ys, want, term_magnitudes(pool, sel, w, xs, H, F))
    # a second call with fewer tokens on the same workspace
    status, ys2, rows2, _ = layer.run(sel[: T // 2 + 1], w[: T // 2 + 1], xs[: T // 2 + 1])
    assert status == 0 and rows2.sum() == (T // 2 + 1) * K
    assert np.array_equal(ys2.view(np.uint32), ys[: T // 2 + 1].view(np.uint32))   # tokens are independent


def test_invalid_selection_publishes_nothing(pkg):
    T, E, K, H, F = 40, 8, 3, 128, 64
    pool = synth.expert_pool(E, H, F, 5)
    sel, w = synth.zipf_selection(T, E, K, 1.1, 6)
    xs = synth.activations(H, T, 7)
    layer = pkg.lib.MoePrefill(pool, E, H, F, K, T)
    untouched = np.full((T, H), 0xFFFFFFFF, np.uint32)
    for kind in ("duplicate", "range", "negative", "nan", "inf"):
        print("prefill invalid", kind, flush=True)
        s2, w2 = sel.copy(), w.copy()
        if kind == "duplicate": s2[4, 1] = s2[4, 0]
        if kind == "range": s2[0, 0] = E
        if kind == "negative": s2[39, 2] = -1
        if kind == "nan": w2[2, 1] = np.nan
        if kind == "inf": w2[7, 0] = -np.inf
        status, ys, _, _ = layer.run(s2, w2, xs)
        assert status == -1 and np.array_equal(ys.view(np.uint32), untouched)
    status, ys, _, _ = layer.run(sel, w, xs)                   # and the layer still works afterwards
    assert status == 0 and np.isfinite(ys).all()
    # without a status word the call itself reports the rejection
    lib = layer.lib
    bad = sel.copy(); bad[1, 1] = bad[1, 0]
    layer.sel.upload(bad)
    rc = lib.salt_mi355_moe_prefill_dev(layer.pool.ptr, layer.stride, H, F, E, K, T, layer.sel.ptr, layer.w.ptr,
                                        layer.x.ptr, layer.out.ptr, None, None, None, layer.ws.ptr,
                                        lib.salt_mi355_stream())
    assert rc == -1 and b"invalid selection" in lib.salt_mi355_last_error()


def test_full_layer_shape_sampled(pkg, oracle):
    """2048 tokens, 128 experts, top-8 of hidden 2816 / routed 704: exact bucketing, sampled values."""
    T, E, K, H, F = 2048, 128, 8, 2816, 704
    print("prefill full layer shape", flush=True)
    pool = synth.expert_pool(E, H, F, 77)
    sel, w = synth.zipf_selection(T, E, K, 1.1, 78)
    xs = synth.activations(H, T, 79)
    layer = pkg.lib.MoePrefill(pool, E, H, F, K, T)
    status, ys, rows, pairs = layer.run(sel, w, xs)
    assert status == 0
    want_rows, want_pairs = expected_grouping(sel, E)
    assert np.array_equal(rows, want_rows) and np.array_equal(pairs, want_pairs)
    g = ExpertGeometry(H, F)
    sample = [0, 1, 777, 1024, 2047]
    want = np.zeros((len(sample), H), np.float32)
    ss, sw, sx = (np.ascontiguousarray(a[sample]) for a in (sel, w, xs))
    assert oracle.orc_moe_group(C.byref(g), ptr(pool), E, K, len(sample), ptr(ss), ptr(sw), ptr(sx), ptr(want), None,
                                host_threads()) == 0
    check_values(ys[sample], want)
    assert np.isfinite(ys).all()
