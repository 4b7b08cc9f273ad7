"""Tolerance-class affine-Q4 decode matvec (salt_mi355_q4_matvec_t_dev, salt_mi355_q4_jobs_t_dev).

The kernel evaluates, per 64-column scale group,  s * sum(q x) + b * sum(x)  with the integer-by-activation sums
exact, so it is not bit-identical to the reference's 32-chain row; its error scales with the magnitudes of the two
terms.  Stated tolerance per output, checked against the bit-exact CPU checker (which the reference's golden
vectors pin):

    |error| <= 2^-20 * sum_c (|q_c s| + 16 |s| + |b|) * |x_c| + 1e-6

and, for activations without outliers, also inside 2^-18 * sum_c |w_c x_c| + 1e-6."""
import ctypes as C

import numpy as np
import pytest

from golden import cases
from oracle_lib import host_threads, ptr

pytestmark = pytest.mark.gpu
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


@pytest.mark.parametrize("R,Cc,B", [
    (4096, 4096, 1),                                   # BASELINE configs[0]
    (2816, 2816, 1), (16384, 2816, 1), (2816, 8192, 1),   # configs[1], batch 1
    (2816, 2816, 4), (16384, 2816, 4), (2816, 8192, 4),   # configs[1], batch 4 (8192 columns: two passes of two tokens)
    (704, 2816, 1), (2816, 704, 1),                    # the experts' projections; 704 columns = 11 groups, an odd count
    (33, 576, 2), (1, 512, 1), (257, 8192, 3), (100, 1024, 7), (31, 640, 9),
])
def test_matvec_within_stated_tolerance(pkg, oracle, R, Cc, B):
    print(f"class T R={R} C={Cc} B={B}", flush=True)
    vals, scales, biases = synth.q4_tensor(R, Cc, 3 * R + Cc + B)
    xs = synth.activations(Cc, B, 23)
    got = pkg.lib.q4_matvec(vals, scales, biases, R, Cc, xs, tolerance_class=True)
    want = reference(oracle, vals, scales, biases, R, Cc, xs)
    check(got, want, vals, scales, biases, R, Cc, xs)


def test_outliers_zeros_and_wide_dynamic_range(pkg, oracle):
    R, Cc = 96, 1024
    vals, scales, biases = synth.q4_tensor(R, Cc, 77)
    xs = synth.activations(Cc, 4, 78)
    xs[0, :6] = [0.0, -0.0, 1e-20, 3e4, -7.5, 1e-38]       # one group spans sixty binades
    xs[1] = 0.0                                          # all zero: every output is +0 or -0
    xs[2] *= np.float32(1e-30)                           # tiny everywhere
    xs[3] *= np.float32(1e20)                            # huge everywhere
    got = pkg.lib.q4_matvec(vals, scales, biases, R, Cc, xs, tolerance_class=True)
    want = reference(oracle, vals, scales, biases, R, Cc, xs)
    assert (got[1] == 0.0).all()
    wx, terms = magnitude_sums(vals, scales, biases, R, Cc, xs)
    err = np.abs(got.astype(np.float64) - want)
    assert (err <= 2.0 ** -20 * terms + 1e-6).all(), float((err / (2.0 ** -20 * terms + 1e-6)).max())
    # the relative part alone holds where the absolute floor of 1e-6 would hide everything
    assert (err[2] <= 2.0 ** -20 * terms[2] + 1e-36).all()


def test_null_bias_pool_alignment_and_exact_fallbacks(pkg, oracle):
    R, Cc = 200, 2816
    vals, scales, biases = synth.q4_tensor(R, Cc, 5)
    xs = synth.activations(Cc, 2, 6)
    got = pkg.lib.q4_matvec(vals, scales, None, R, Cc, xs, tolerance_class=True)
    check(got, reference(oracle, vals, scales, None, R, Cc, xs), vals, scales, None, R, Cc, xs)
    # the engine's expert pool file puts every tensor 8 bytes past a multiple of 16
    for offset in (8, 4):
        got = pkg.lib.q4_matvec(vals, scales, biases, R, Cc, xs, value_offset=offset, tolerance_class=True)
        check(got, reference(oracle, vals, scales, biases, R, Cc, xs), vals, scales, biases, R, Cc, xs)
    # shapes the streaming kernel does not take run on the bit-exact kernels: equal bits
    for r, c in ((40, 448), (7, 200), (64, 64)):
        pad = (-(r * c)) % 64
        v, s, b = synth.q4_tensor(1, r * c + pad, 9)
        x = synth.activations(c, 2, 10)
        got = pkg.lib.q4_matvec(v, s, b, r, c, x, tolerance_class=True)
        want = np.zeros((2, r), np.float32)
        assert oracle.orc_q4_matvec_batch(ptr(v), ptr(s), ptr(b), r, c, 2, ptr(x), ptr(want)) == 0
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    got = pkg.lib.q4_matvec(vals, scales, biases, R, Cc, xs, value_offset=1, tolerance_class=True)   # byte-misaligned
    want = reference(oracle, vals, scales, biases, R, Cc, xs)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_non_finite_activation_gives_non_finite_outputs(pkg):
    R, Cc = 64, 512
    vals, scales, biases = synth.q4_tensor(R, Cc, 31)
    xs = synth.activations(Cc, 3, 32)
    xs[0, 100] = np.nan
    xs[2, 511] = np.inf
    got = pkg.lib.q4_matvec(vals, scales, biases, R, Cc, xs, tolerance_class=True)
    assert not np.isfinite(got[0]).any() and not np.isfinite(got[2]).any()
    assert np.isfinite(got[1]).all()


def test_many_jobs_one_launch(pkg, oracle):
    lib = pkg.lib.init()
    Cc, tokens = 2816, 2
    rows = [704, 33, 2816, 256, 1, 300]
    held, jobs, expect = [], (pkg.lib.Q4Job * len(rows))(), []
    for j, R in enumerate(rows):
        vals, scales, biases = synth.q4_tensor(R, Cc, 100 + j)
        xs = synth.activations(Cc, tokens, 200 + j)
        dv, ds, db, dx = (pkg.lib.DeviceBuffer.from_host(a) for a in (vals, scales, biases, xs))
        dy = pkg.lib.DeviceBuffer(tokens * R * 4, fill=0xFF)
        held.append((dv, ds, db, dx, dy))
        jobs[j] = pkg.lib.Q4Job(dv.ptr, ds.ptr, db.ptr, dx.ptr, dy.ptr, R)
        expect.append((vals, scales, biases, R, xs))
    stream = lib.salt_mi355_stream()
    pkg.lib.check(lib.salt_mi355_q4_jobs_t_dev(jobs, len(rows), Cc, tokens, stream), "q4_jobs_t_dev")
    pkg.lib.check(lib.salt_mi355_stream_sync(stream), "sync")
    for (dv, ds, db, dx, dy), (vals, scales, biases, R, xs) in zip(held, expect):
        got = dy.to_host(np.float32).reshape(tokens, R)
        check(got, reference(oracle, vals, scales, biases, R, Cc, xs), vals, scales, biases, R, Cc, xs)


@pytest.mark.parametrize("R,Cc,njobs,tokens", [(2816, 2816, 24, 1), (2816, 2816, 24, 3), (8192, 8192, 8, 1), (1424, 704, 48, 2)])
def test_launches_with_many_blocks_take_the_sixteen_row_shape(pkg, oracle, R, Cc, njobs, tokens):
    """From 2048 blocks of 32 rows on, a launch runs on q4_dot16_kernel (16 rows per wave).  Three weight tensors are
    shared by the jobs; every job has its own activations and outputs."""
    lib = pkg.lib.init()
    tensors = [synth.q4_tensor(R, Cc, 500 + k) for k in range(3)]
    dev = [tuple(pkg.lib.DeviceBuffer.from_host(a) for a in t) for t in tensors]
    xs = [synth.activations(Cc, tokens, 600 + j) for j in range(njobs)]
    dxs = [pkg.lib.DeviceBuffer.from_host(x) for x in xs]
    dys = [pkg.lib.DeviceBuffer(tokens * R * 4, fill=0xFF) for _ in range(njobs)]
    jobs = (pkg.lib.Q4Job * njobs)()
    for j in range(njobs):
        dv, ds, db = dev[j % 3]
        jobs[j] = pkg.lib.Q4Job(dv.ptr, ds.ptr, db.ptr, dxs[j].ptr, dys[j].ptr, R)
    stream = lib.salt_mi355_stream()
    pkg.lib.check(lib.salt_mi355_q4_jobs_t_dev(jobs, njobs, Cc, tokens, stream), "q4_jobs_t_dev")
    pkg.lib.check(lib.salt_mi355_stream_sync(stream), "sync")
    assert lib.salt_mi355_last_kernel().decode().startswith("q4_dot16_kernel"), lib.salt_mi355_last_kernel()
    for j in range(0, njobs, 5):
        vals, scales, biases = tensors[j % 3]
        got = dys[j].to_host(np.float32).reshape(tokens, R)
        check(got, reference(oracle, vals, scales, biases, R, Cc, xs[j]), vals, scales, biases, R, Cc, xs[j])


def test_rejections(pkg):
    lib = pkg.lib.init()
    buf = pkg.lib.DeviceBuffer(1 << 16)
    assert lib.salt_mi355_q4_matvec_t_dev(None, buf.ptr, None, 8, 512, 1, buf.ptr, buf.ptr, None) == -1
    assert lib.salt_mi355_q4_matvec_t_dev(buf.ptr, buf.ptr, None, 0, 512, 1, buf.ptr, buf.ptr, None) == -1
    assert lib.salt_mi355_q4_jobs_t_dev(None, 1, 512, 1, None) == -1
