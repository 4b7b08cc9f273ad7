"""The stated tolerance of the tolerance-class affine-Q4 kernels, shared by their tests: per output

    |error| <= 2^-20 * sum_c (|q_c s| + 16 |s| + |b|) * |x_c| + 1e-6

against the bit-exact CPU checker and, for activations without outliers, also 2^-18 * sum_c |w_c x_c| + 1e-6."""
import numpy as np

from golden import cases
from oracle_lib import host_threads, ptr

synth = cases.synth


def reference(oracle, vals, scales, biases, R, Cc, xs):
    ys = np.zeros((xs.shape[0], R), np.float32)
    for t in range(xs.shape[0]):
        assert oracle.orc_q4_matvec_threads(ptr(vals), ptr(scales), ptr(biases), R, Cc, ptr(xs[t]), ptr(ys[t]),
                                            host_threads()) == 0
    return ys


def magnitude_sums(vals, scales, biases, R, Cc, xs):
    """(sum_c |w x|, sum_c (|q s| + 16|s| + |b|) |x|) per (token, row), in float64, row blocks to bound memory."""
    wx = np.zeros((xs.shape[0], R))
    terms = np.zeros((xs.shape[0], R))
    ax = np.abs(xs.astype(np.float64))
    words = vals.reshape(R, Cc // 8)
    sc = synth.bf16_bits_to_f32(scales).reshape(R, Cc // 64).astype(np.float64)
    bi = np.zeros((R, Cc // 64)) if biases is None else synth.bf16_bits_to_f32(biases).reshape(R, Cc // 64).astype(np.float64)
    for r0 in range(0, R, 1024):
        r1 = min(R, r0 + 1024)
        q = ((words[r0:r1, :, None] >> (4 * np.arange(8, dtype=np.uint32))) & 15).reshape(r1 - r0, Cc).astype(np.float64)
        s = np.repeat(sc[r0:r1], 64, axis=1)
        b = np.repeat(bi[r0:r1], 64, axis=1)
        wx[:, r0:r1] = ax @ np.abs(q * s + b).T
        terms[:, r0:r1] = ax @ (np.abs(q * s) + 16 * np.abs(s) + np.abs(b)).T
    return wx, terms


def check(got, want, vals, scales, biases, R, Cc, xs, outlier_tokens=()):
    wx, terms = magnitude_sums(vals, scales, biases, R, Cc, xs)
    err = np.abs(got.astype(np.float64) - want)
    bound = 2.0 ** -20 * terms + 1e-6
    assert np.isfinite(got).all()
    print("max err / bound", float((err / bound).max()), flush=True)
    assert (err <= bound).all(), float((err / bound).max())
    plain = 2.0 ** -18 * wx + 1e-6
    keep = [t for t in range(xs.shape[0]) if t not in outlier_tokens]
    if keep:
        print("max err / plain bound", float((err[keep] / plain[keep]).max()), flush=True)
        assert (err[keep] <= plain[keep]).all()
