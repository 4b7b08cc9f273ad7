"""Prefill-sized affine-Q4 matmul on the matrix cores: tolerance class.

The kernel evaluates the affine form per scale group, s * sum(q x) + b * sum(x),
so its rounding error scales with the magnitudes of the two terms, not with
their (possibly cancelling) sum.  Stated tolerance per output, checked against
the bit-exact CPU checker:

    |error| <= 2^-20 * sum_c (|q_c s| + 16 |s| + |b|) * |x_c| + 1e-6

For activations without outliers this is also inside 2^-18 * sum_c |w_c x_c|,
which the second assertion checks on plain N(0,1) inputs."""
import numpy as np
import pytest

from golden import cases
from oracle_lib import host_threads, ptr

pytestmark = pytest.mark.gpu
synth = cases.synth


def reference(oracle, vals, scales, biases, R, C, xs):
    ys = np.zeros((xs.shape[0], R), np.float32)
    for t in range(xs.shape[0]):
        assert oracle.orc_q4_matvec_threads(ptr(vals), ptr(scales), ptr(biases), R, C, ptr(xs[t]), ptr(ys[t]),
                                            host_threads()) == 0
    return ys


def magnitude_sums(vals, scales, biases, R, C, xs):
    """(sum_c |w x|, sum_c (|q s| + 16|s| + |b|) |x|) per (token, row)."""
    q = ((vals[:, None] >> (4 * np.arange(8, dtype=np.uint32))) & 15).reshape(R, C).astype(np.float64)
    s = np.repeat(synth.bf16_bits_to_f32(scales).reshape(R, C // 64), 64, axis=1).astype(np.float64)
    b = np.zeros((R, C)) if biases is None else np.repeat(synth.bf16_bits_to_f32(biases).reshape(R, C // 64), 64, axis=1)
    ax = np.abs(xs.astype(np.float64))
    return ax @ np.abs(q * s + b).T, ax @ (np.abs(q * s) + 16 * np.abs(s) + np.abs(b)).T


@pytest.mark.parametrize("R,C,B", [(64, 64, 64), (128, 256, 32), (704, 2816, 100), (2816, 704, 37), (70, 128, 1), (33, 192, 130)])
def test_matmul_within_stated_tolerance(pkg, oracle, R, C, B):
    print(f"mfma R={R} C={C} B={B}", flush=True)
    vals, scales, biases = synth.q4_tensor(R, C, R + C + B)
    xs = synth.activations(C, B, 17)
    xs[0, :5] = [0.0, -0.0, 1e-20, 3e4, -7.5]
    got = pkg.lib.q4_matmul(vals, scales, biases, R, C, xs)
    want = reference(oracle, vals, scales, biases, R, C, xs)
    wx, terms = magnitude_sums(vals, scales, biases, R, C, xs)
    bound = 2.0 ** -20 * terms + 1e-6
    err = np.abs(got.astype(np.float64) - want)
    assert np.isfinite(got).all()
    print("max err / bound", float((err / bound).max()), flush=True)
    assert (err <= bound).all(), float((err / bound).max())
    plain = 2.0 ** -18 * wx[1:] + 1e-6            # token 0 carries the outliers
    if B > 1:
        print("max err / plain bound", float((err[1:] / plain).max()), flush=True)
        assert (err[1:] <= plain).all()


def test_matmul_null_bias_and_rejections(pkg, oracle):
    vals, scales, _ = synth.q4_tensor(64, 128, 3)
    xs = synth.activations(128, 16, 4)
    got = pkg.lib.q4_matmul(vals, scales, None, 64, 128, xs)
    want = reference(oracle, vals, scales, None, 64, 128, xs)
    assert (np.abs(got - want) <= 2.0 ** -20 * magnitude_sums(vals, scales, None, 64, 128, xs)[1] + 1e-6).all()
    lib = pkg.lib.init()
    buf = pkg.lib.DeviceBuffer(1 << 16)
    assert lib.salt_mi355_q4_matmul_dev(buf.ptr, buf.ptr, None, 8, 96, 4, buf.ptr, buf.ptr, buf.ptr, None) == -1   # C % 64
    assert lib.salt_mi355_q4_matmul_workspace_bytes(96, 4) == 0
