"""Tolerance-class MoE decode layer-step (salt_mi355_moe_decode_step_t_dev).

Router top-k, selection and routing weights are bit-identical to the reference (same code as the bit-exact step); the
expert projections run on the tolerance-class matvec kernel, so expert outputs and the layer output carry a stated
tolerance against the bit-exact CPU checker:

    |expert_out[e][d] - ref| <= 2^-15 * max_d |ref[e]| + 1e-6        |out[d] - ref| <= 2^-15 * max_d |ref| + 1e-6"""
import ctypes as C

import numpy as np
import pytest

from golden import cases
from oracle_lib import ExpertGeometry, bits, ptr

pytestmark = pytest.mark.gpu
synth = cases.synth


def run(pkg, oracle, E, K, H, F, pool_seed, logit_seed, x_seed, header=0):
    pool = synth.expert_pool(E, H, F, pool_seed)
    layer = pkg.lib.MoeLayer(pool, E, H, F, K, header_bytes=header)
    layer.tolerance_class = True
    logits, scale = synth.router_logits(E, logit_seed), (1.0 + 0.1 * synth.router_logits(E, logit_seed + 1)).astype(np.float32)
    x = synth.activations(H, 1, x_seed)[0]
    status, sel, w, eo, y = layer.step(logits, scale, x)
    g = ExpertGeometry(H, F)
    osel, ow = np.zeros(K, np.int32), np.zeros(K, np.float32)
    oeo, oy = np.zeros((K, H), np.float32), np.zeros(H, np.float32)
    assert oracle.orc_moe_decode_step(C.byref(g), ptr(pool), E, K, ptr(logits), ptr(scale), ptr(x), ptr(osel), ptr(ow),
                                      ptr(oeo), ptr(oy), 2) == 0
    assert status == 0 and np.array_equal(sel, osel) and np.array_equal(bits(w), bits(ow))
    bound_e = 2.0 ** -15 * np.abs(oeo).max(axis=1, keepdims=True) + 1e-6
    ratio_e = float((np.abs(eo.astype(np.float64) - oeo) / bound_e).max())
    bound_y = 2.0 ** -15 * np.abs(oy).max() + 1e-6
    ratio_y = float((np.abs(y.astype(np.float64) - oy) / bound_y).max())
    print(f"E={E} K={K} H={H} F={F}: expert_out err/bound {ratio_e:.3f}, out err/bound {ratio_y:.3f}", flush=True)
    assert ratio_e <= 1.0 and ratio_y <= 1.0
    return layer


@pytest.mark.parametrize("E,K,H,F", [(128, 8, 2816, 704), (16, 8, 2816, 704), (8, 3, 512, 512), (200, 1, 1024, 640)])
def test_step_within_stated_tolerance(pkg, oracle, E, K, H, F):
    run(pkg, oracle, E, K, H, F, 21, 621, 622)


def test_pool_file_header_alignment_and_consecutive_steps(pkg, oracle):
    layer = run(pkg, oracle, 16, 8, 2816, 704, 23, 631, 632, header=24)      # tensors 8 bytes past a multiple of 16
    for k in range(5):
        logits = synth.router_logits(16, 700 + k)
        x = synth.activations(2816, 1, 710 + k)[0]
        status, sel, w, eo, y = layer.step(logits, np.ones(16, np.float32), x)
        assert status == 0 and np.isfinite(y).all() and len(set(sel.tolist())) == 8


def test_rejected_router_input_publishes_nothing(pkg):
    E, K, H, F = 16, 4, 512, 512
    pool = synth.expert_pool(E, H, F, 5)
    layer = pkg.lib.MoeLayer(pool, E, H, F, K)
    layer.tolerance_class = True
    layer.out.upload(np.full(H, 7.0, np.float32))
    logits = synth.router_logits(E, 6)
    logits[3] = np.nan
    status, sel, w, eo, y = layer.step(logits, np.ones(E, np.float32), synth.activations(H, 1, 7)[0])
    assert status == -1 and (y == 7.0).all()


def test_geometries_outside_the_streaming_kernel_take_the_exact_plan(pkg, oracle):
    # 64-wide experts (below 512 columns) and more than 256 experts: bit-exact results through the same entry point
    for E, K, H, F in ((8, 3, 256, 128), (300, 4, 512, 512)):
        pool = synth.expert_pool(E, H, F, 31)
        layer = pkg.lib.MoeLayer(pool, E, H, F, K)
        layer.tolerance_class = True
        logits, scale = synth.router_logits(E, 32), np.ones(E, np.float32)
        x = synth.activations(H, 1, 33)[0]
        status, sel, w, eo, y = layer.step(logits, scale, x)
        g = ExpertGeometry(H, F)
        osel, ow = np.zeros(K, np.int32), np.zeros(K, np.float32)
        oeo, oy = np.zeros((K, H), np.float32), np.zeros(H, np.float32)
        assert oracle.orc_moe_decode_step(C.byref(g), ptr(pool), E, K, ptr(logits), ptr(scale), ptr(x), ptr(osel),
                                          ptr(ow), ptr(oeo), ptr(oy), 2) == 0
        assert status == 0 and np.array_equal(sel, osel)
        assert np.array_equal(bits(y), bits(oy)) and np.array_equal(bits(eo), bits(oeo))


def test_router_ties_zeros_and_all_equal_logits_choose_the_reference_experts(pkg, oracle):
    """The gate/up launch finds its experts with a wave-level search of its own: ties must go to the smaller index,
    -0 and +0 are one value, all-equal logits select the first topk experts."""
    E, K, H, F = 128, 8, 512, 512
    pool = synth.expert_pool(E, H, F, 41)
    layer = pkg.lib.MoeLayer(pool, E, H, F, K)
    layer.tolerance_class = True
    g = ExpertGeometry(H, F)
    x = synth.activations(H, 1, 42)[0]
    scale = np.ones(E, np.float32)
    rng = synth.rng(43)
    cases_ = [np.zeros(E, np.float32), np.full(E, -3.5, np.float32),
              rng.integers(-2, 3, E).astype(np.float32),                       # five distinct values: many ties
              np.where(np.arange(E) % 2 == 0, np.float32(0.0), np.float32(-0.0)).astype(np.float32),
              np.concatenate([np.full(E - 3, 1.0), [2.0, 1.0, 2.0]]).astype(np.float32),
              -np.abs(synth.router_logits(E, 44))]
    for logits in cases_:
        status, sel, w, eo, y = layer.step(logits, scale, x)
        osel, ow = np.zeros(K, np.int32), np.zeros(K, np.float32)
        oeo, oy = np.zeros((K, H), np.float32), np.zeros(H, np.float32)
        assert oracle.orc_moe_decode_step(C.byref(g), ptr(pool), E, K, ptr(logits), ptr(scale), ptr(x), ptr(osel),
                                          ptr(ow), ptr(oeo), ptr(oy), 2) == 0
        assert status == 0 and np.array_equal(sel, osel) and np.array_equal(bits(w), bits(ow))
        # expert_out rows are in selection order: a wrong expert in any workgroup would show as a large error
        bound = 2.0 ** -15 * np.abs(oeo).max(axis=1, keepdims=True) + 1e-6
        assert (np.abs(eo.astype(np.float64) - oeo) <= bound).all()
