"""Tolerance-class MoE decode layer-step (salt_mi355_moe_decode_step_t_dev).

Router top-k, selection and routing weights are bit-identical to the reference (same code as the bit-exact step); the
expert projections run on the tolerance-class matvec kernels, so expert outputs and the layer output carry a stated
tolerance against the bit-exact CPU checker, per output and relative to the sum of the magnitudes of its terms:

    |expert_out[k][d] - ref| <= 2^-18 * sum_f |Wd_k[d][f] * h_k[f]| + 1e-6
    |out[d] - ref|           <= 2^-18 * sum_k |w_k| * sum_f |Wd_k[d][f] * h_k[f]| + 1e-6

with h_k = gelu_tanh(gate_k) * up_k the expert's activation and Wd_k its dequantised down projection (float64, computed
here).  The tests also pin which launch plan served each geometry (salt_mi355_last_kernel): a plan that silently fell
back to another would still be inside the bound."""
import ctypes as C

import numpy as np
import pytest

from golden import cases
from moe_bounds import down_term_magnitudes, expert_activation
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
    ratio_e, ratio_y = error_ratios(pool, H, F, x, osel, ow, eo, y, oeo, oy)
    print(f"E={E} K={K} H={H} F={F}: expert_out err/bound {ratio_e:.3f}, out err/bound {ratio_y:.3f}", flush=True)
    assert ratio_e <= 1.0 and ratio_y <= 1.0
    return layer


def error_ratios(pool, H, F, x, sel, w, eo, y, want_eo, want_y):
    """Largest error / bound over the expert outputs and over the layer output (bounds of the module docstring)."""
    terms = np.stack([down_term_magnitudes(pool, e, expert_activation(pool, e, x[None, :], H, F), H, F)[0] for e in sel])
    bound_e = 2.0 ** -18 * terms + 1e-6
    bound_y = 2.0 ** -18 * (np.abs(w.astype(np.float64))[:, None] * terms).sum(axis=0) + 1e-6
    return (float((np.abs(eo.astype(np.float64) - want_eo) / bound_e).max()),
            float((np.abs(y.astype(np.float64) - want_y) / bound_y).max()))


# the launch plan that serves each geometry: two launches on the sixteen-row stream where it fits, else gate/up,
# down and the sum as three launches on the 32-row kernel (more than 128 experts with one part per matrix)
PLAN = {(128, 8, 2816, 704): "moe16_gate_up_kernel<3,4> + moe16_down_sum_kernel<4>",
        (16, 8, 2816, 704): "moe16_gate_up_kernel<3,4> + moe16_down_sum_kernel<4>",
        (8, 3, 512, 512): "moe16_gate_up_kernel<1,4> + moe16_down_sum_kernel<4>",
        (200, 1, 1024, 640): "q4_dot_kernel<1,4,2,16,2> ksplit 2",
        (64, 4, 4096, 2048): "moe16_gate_up_kernel<3,8> + moe16_down_sum_kernel<8>",
        (32, 2, 1536, 2560): "moe16_gate_up_kernel<3,4> + moe16_down_sum_kernel<16>",
        (8, 2, 6272, 512): "moe16_gate_up_kernel<3,16> + moe16_down_sum_kernel<4>"}


@pytest.mark.parametrize("E,K,H,F", list(PLAN))
def test_step_within_stated_tolerance(pkg, oracle, E, K, H, F):
    run(pkg, oracle, E, K, H, F, 21, 621, 622)
    assert pkg.lib.init().salt_mi355_last_kernel().decode() == PLAN[(E, K, H, F)]


def test_same_call_gives_the_same_bits(pkg):
    """No atomics and no launch-order dependence in either launch: a step repeated on the same inputs, before and
    after other work on the device, returns identical bits."""
    E, K, H, F = 128, 8, 2816, 704
    pool = synth.expert_pool(E, H, F, 51)
    layer = pkg.lib.MoeLayer(pool, E, H, F, K)
    layer.tolerance_class = True
    logits, scale, x = synth.router_logits(E, 52), np.ones(E, np.float32), synth.activations(H, 1, 53)[0]
    first = layer.step(logits, scale, x)
    other = layer.step(synth.router_logits(E, 54), scale, synth.activations(H, 1, 55)[0])
    assert not np.array_equal(first[1], other[1])                      # a different selection ran in between
    for _ in range(3):
        again = layer.step(logits, scale, x)
        assert again[0] == 0 and np.array_equal(again[1], first[1])
        for a, b in zip(again[2:], first[2:]):
            assert np.array_equal(bits(a), bits(b))


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
        ratio_e, ratio_y = error_ratios(pool, H, F, x, osel, ow, eo, y, oeo, oy)
        assert ratio_e <= 1.0 and ratio_y <= 1.0
