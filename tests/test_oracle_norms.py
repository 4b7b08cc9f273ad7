"""CPU checker for the norms and residual combinations around the MoE step (rmsnorm, router input, residual post-norm,
parallel combine, softcap) and their square roots: pinned by the reference's own compiled functions, by closed forms and
by libm."""
import math

import numpy as np
import pytest

from golden import cases
from oracle_lib import bits, ptr

synth = cases.synth
f32 = np.float32


def ulp_distance(a, b):
    ia = np.asarray(a, f32).view(np.int32).astype(np.int64); ib = np.asarray(b, f32).view(np.int32).astype(np.int64)
    return np.abs(ia - ib)


def test_square_roots_closed_forms_and_libm(oracle):
    for k in range(-60, 61):
        x = f32(4.0) ** k
        assert oracle.orc_rsqrtf(x) == f32(2.0) ** (-k) and oracle.orc_sqrtf(x) == f32(2.0) ** k
    g = synth.rng(1)
    xs = np.exp(g.uniform(-80, 80, 4000)).astype(f32)
    got_r = np.array([oracle.orc_rsqrtf(x) for x in xs], f32)
    got_s = np.array([oracle.orc_sqrtf(x) for x in xs], f32)
    # the double Newton result rounded once: the correctly rounded value, or its neighbour at a double rounding
    assert ulp_distance(got_r, (1.0 / np.sqrt(xs.astype(np.float64))).astype(f32)).max() <= 1
    assert ulp_distance(got_s, np.sqrt(xs.astype(np.float64)).astype(f32)).max() <= 1
    assert math.isnan(oracle.orc_rsqrtf(f32(-1.0))) and oracle.orc_rsqrtf(f32(0.0)) == math.inf
    assert oracle.orc_sqrtf(f32(0.0)) == 0.0 and math.isnan(oracle.orc_sqrtf(f32(-4.0)))
    tiny = f32(2.0) ** -140                                     # subnormal input: the rescaled branch
    assert oracle.orc_rsqrtf(tiny) == f32(2.0) ** 70 and oracle.orc_sqrtf(tiny) == f32(2.0) ** -70
    assert oracle.orc_pow_minus_half(f32(0.0)) == 0.0 and oracle.orc_pow_minus_half(f32(1.0)) == 1.0


def test_square_roots_equal_compiled_reference(oracle, reference):
    g = synth.rng(2)
    xs = np.concatenate([np.exp(g.uniform(-100, 88, 20000)).astype(f32),
                         np.array([0.0, 1.0, 2.0 ** -126, 2.0 ** -149, 3.4e38, np.inf], f32)])
    for x in xs:
        a, b = oracle.orc_rsqrtf(x), reference.salt_rsqrtf(x)
        assert bits(f32(a)) == bits(f32(b)) or (math.isnan(a) and math.isnan(b)), x
        a, b = oracle.orc_sqrtf(x), reference.salt_sqrtf(x)
        assert bits(f32(a)) == bits(f32(b)) or (math.isnan(a) and math.isnan(b)), x
        a, b = oracle.orc_pow_minus_half(x), reference.salt_powf(x, f32(-0.5))
        assert bits(f32(a)) == bits(f32(b)) or (math.isnan(a) and math.isnan(b)), x


def test_rmsnorm_closed_forms(oracle):
    n = 1024
    x = np.full(n, 8.0, f32); x[::2] = -8.0
    w = np.full(n, 0.5, f32); out = np.zeros(n, f32)
    assert oracle.orc_rmsnorm(ptr(out), ptr(x), ptr(w), n, 0.0, 1) == 0          # mean square 64 -> inv = 1/8 exactly
    assert np.array_equal(out, np.where(x > 0, 0.5, -0.5).astype(f32))
    assert oracle.orc_rmsnorm(ptr(out), ptr(x), None, n, 0.0, 0) == 0 and np.array_equal(np.abs(out), np.ones(n, f32))
    # the sum of squares is one left-to-right chain: 2^24 followed by ones stays 2^24 (a tree would not)
    n = 4096
    x = np.ones(n, f32); x[0] = 4096.0
    assert oracle.orc_rmsnorm(ptr(out := np.zeros(n, f32)), ptr(x), None, n, 0.0, 0) == 0
    inv = oracle.orc_rsqrtf(f32(f32(2.0 ** 24) / f32(n)))
    assert np.array_equal(bits(out), bits((x * f32(inv)).astype(f32)))
    # rejection: non-finite input, negative eps, partial overlap; exact aliasing is allowed
    bad = x.copy(); bad[7] = np.inf
    assert oracle.orc_rmsnorm(ptr(out), ptr(bad), None, n, 0.0, 0) == -1
    assert oracle.orc_rmsnorm(ptr(out), ptr(x), None, n, -1.0, 0) == -1
    buf = np.ones(n + 8, f32)
    assert oracle.orc_rmsnorm(ptr(buf[8:]), ptr(buf[:n]), None, n, 1e-6, 0) == -1
    assert oracle.orc_rmsnorm(ptr(buf[:n]), ptr(buf[:n]), None, n, 1e-6, 0) == 0


@pytest.mark.parametrize("n,seed", [(2816, 3), (64, 4), (1, 5), (4097, 6)])
def test_norm_family_equals_compiled_reference(oracle, reference, n, seed):
    g = synth.rng(seed)
    mk = lambda s: (g.standard_normal(n) * s).astype(f32)
    x, w, w2, w3, res, dense, routed = mk(3), mk(1), mk(1), mk(1), mk(2), mk(5), mk(0.01)
    eps = f32(1e-6)
    for with_scale in (0, 1):
        a = np.zeros(n, f32); b = np.zeros(n, f32)
        assert oracle.orc_rmsnorm(ptr(a), ptr(x), ptr(w), n, eps, with_scale) == 0
        assert reference.salt_gemma4_rmsnorm(ptr(b), ptr(x), ptr(w), n, eps, with_scale) == 0
        assert np.array_equal(bits(a), bits(b))
    a = np.zeros(n, f32); b = np.zeros(n, f32)
    assert oracle.orc_router_input(ptr(a), ptr(x), ptr(w), n, eps) == 0
    assert reference.salt_gemma4_router_input(ptr(b), ptr(x), ptr(w), n, eps) == 0
    assert np.array_equal(bits(a), bits(b))
    assert oracle.orc_residual_postnorm(ptr(a), ptr(res), ptr(x), ptr(w), n, eps) == 0
    assert reference.salt_gemma4_residual_postnorm(ptr(b), ptr(res), ptr(x), ptr(w), n, eps) == 0
    assert np.array_equal(bits(a), bits(b))
    scratch = np.zeros(2 * n, f32)
    assert oracle.orc_parallel_ffn_combine(ptr(a), ptr(res), ptr(dense), ptr(routed), ptr(w), ptr(w2), ptr(w3), f32(0.37), n,
                                           eps) == 0
    assert reference.salt_gemma4_parallel_ffn_combine(ptr(b), ptr(res), ptr(dense), ptr(routed), ptr(w), ptr(w2), ptr(w3),
                                                      f32(0.37), n, eps, ptr(scratch)) == 0
    assert np.array_equal(bits(a), bits(b))
    logits = mk(40); l2 = logits.copy()
    assert oracle.orc_softcap(ptr(logits), n, f32(30.0)) == 0 and reference.salt_gemma4_softcap(ptr(l2), n, f32(30.0)) == 0
    assert np.array_equal(bits(logits), bits(l2))
    # both reject the same things and leave the output alone
    bad = dense.copy(); bad[n // 2] = np.nan
    a[:] = 7.0; b[:] = 7.0
    assert oracle.orc_parallel_ffn_combine(ptr(a), ptr(res), ptr(bad), ptr(routed), ptr(w), ptr(w2), ptr(w3), f32(1.0), n,
                                           eps) == -1
    assert reference.salt_gemma4_parallel_ffn_combine(ptr(b), ptr(res), ptr(bad), ptr(routed), ptr(w), ptr(w2), ptr(w3),
                                                      f32(1.0), n, eps, ptr(scratch)) == -1
    assert (a == 7.0).all() and (b == 7.0).all()
    assert oracle.orc_softcap(ptr(logits), n, f32(0.0)) == -1 and reference.salt_gemma4_softcap(ptr(l2), n, f32(0.0)) == -1


def test_combine_and_softcap_closed_forms(oracle):
    n = 256
    ones = np.ones(n, f32)
    dense = np.full(n, 4.0, f32); routed = np.full(n, -2.0, f32); res = np.arange(n, dtype=f32)
    out = np.zeros(n, f32)
    # norm(dense) = 1, norm(routed) = -1 -> sum 0 -> its norm is 0 * pow(0, -0.5) = 0 * 0 -> out = residual * scalar
    assert oracle.orc_parallel_ffn_combine(ptr(out), ptr(res), ptr(dense), ptr(routed), ptr(ones), ptr(ones), ptr(ones),
                                           f32(0.5), n, 0.0) == 0
    assert np.array_equal(out, res * f32(0.5))
    # weights 3 and 1: sum = 3 - 1 = 2 everywhere, final norm = 1, out = (res + 1) * 2
    assert oracle.orc_parallel_ffn_combine(ptr(out), ptr(res), ptr(dense), ptr(routed), ptr(ones * 3), ptr(ones), ptr(ones),
                                           f32(2.0), n, 0.0) == 0
    assert np.array_equal(out, (res + 1) * 2)
    z = np.zeros(4, f32)
    assert oracle.orc_softcap(ptr(z), 4, f32(30.0)) == 0 and (z == 0).all()
    big = np.array([1e6, -1e6, 300.0, -300.0], f32)
    assert oracle.orc_softcap(ptr(big), 4, f32(30.0)) == 0 and np.array_equal(big, np.array([30, -30, 30, -30], f32))


@pytest.mark.parametrize("H,D,F,E,K,seed", [(256, 192, 128, 16, 4, 1), (2816, 2112, 704, 8, 3, 2)])
def test_ffn_block_equals_the_reference_functions_in_the_engine_order(oracle, reference, H, D, F, E, K, seed):
    """feed_forward itself is a static function of the model file; its public constituents from the compiled
    reference are driven here in its order (gemma4_text.c:8308-8390, routed_experts 7908-8306)."""
    import ctypes as C
    from oracle_lib import ffn_layer_struct
    w = synth.ffn_layer(H, D, F, E, K, seed)
    L = ffn_layer_struct(w)
    residual = (synth.activations(H, 1, 50 + seed)[0] * 3).astype(f32)
    out = np.zeros(H, f32); sel = np.zeros(K, np.int32); wt = np.zeros(K, f32)
    assert oracle.orc_ffn_block(C.byref(L), ptr(residual), ptr(out), ptr(sel), ptr(wt), 4) == 0
    eps = w["eps"]
    r = reference
    q4 = lambda t, R, Cc, x: (y := np.zeros(R, f32), r.salt_q4_matvec(ptr(t[0]), ptr(t[1]), ptr(t[2]), R, Cc, ptr(x), ptr(y)))[0]
    norm_a = np.zeros(H, f32)
    assert r.salt_gemma4_rmsnorm(ptr(norm_a), ptr(residual), ptr(w["pre_norm"]), H, eps, 1) == 0
    gate, up = q4(w["dense_gate"], D, H, norm_a), q4(w["dense_up"], D, H, norm_a)
    act = np.array([f32(r.salt_gemma4_gelu_tanh(a)) * b for a, b in zip(gate, up)], f32)
    dense_out = q4(w["dense_down"], H, D, act)
    router_in = np.zeros(H, f32)
    assert r.salt_gemma4_router_input(ptr(router_in), ptr(residual), ptr(w["router_scale"]), H, eps) == 0
    logits = np.zeros(E, f32)
    r.salt_q8_matvec(ptr(w["router"][0]), ptr(w["router"][1]), ptr(w["router"][2]), E, H, ptr(router_in), ptr(logits))
    rsel = np.zeros(K, np.int32); rw = np.zeros(K, f32)
    assert r.salt_gemma4_router_topk(ptr(logits), ptr(w["per_expert_scale"]), E, K, ptr(rsel), ptr(rw)) == 0
    order = np.argsort(rsel, kind="stable"); rsel, rw = rsel[order], rw[order]
    norm_b = np.zeros(H, f32)
    assert r.salt_gemma4_rmsnorm(ptr(norm_b), ptr(residual), ptr(w["pre_norm_2"]), H, eps, 1) == 0
    routed = np.zeros(H, f32)
    for e, weight in zip(rsel, rw):
        views = [synth.expert_views(w["pool"], int(e), p, H, F) for p in range(3)]
        g1, u1 = q4(views[0], F, H, norm_b), q4(views[1], F, H, norm_b)
        h = np.array([f32(r.salt_gemma4_gelu_tanh(a)) * b for a, b in zip(g1, u1)], f32)
        o = q4(views[2], H, F, h)
        routed = (routed + (o * weight).astype(f32)).astype(f32)
    want = np.zeros(H, f32); scratch = np.zeros(2 * H, f32)
    assert r.salt_gemma4_parallel_ffn_combine(ptr(want), ptr(residual), ptr(dense_out), ptr(routed), ptr(w["post_norm_1"]),
                                              ptr(w["post_norm_2"]), ptr(w["post_norm"]), w["layer_scalar"], H, eps,
                                              ptr(scratch)) == 0
    assert np.array_equal(sel, rsel) and np.array_equal(bits(wt), bits(rw))
    assert np.array_equal(bits(out), bits(want))
    assert len(set(np.round(logits, 6))) == E                   # the routing is not decided by ties
