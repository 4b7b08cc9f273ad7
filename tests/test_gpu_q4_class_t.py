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
from oracle_lib import ptr
from q4_bounds import check, magnitude_sums, reference

pytestmark = pytest.mark.gpu
synth = cases.synth


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


def run_jobs(pkg, Cc, tokens, rows, weights, seed):
    """One salt_mi355_q4_jobs_t_dev launch of len(rows) jobs; job j reads weights[j % len(weights)] (tensors of at
    least rows[j] rows) and its own activations.  Returns (kernel name, [(tensor, rows, xs, ys)])."""
    lib = pkg.lib.init()
    dev = [tuple(pkg.lib.DeviceBuffer.from_host(a) for a in t) for t in weights]
    xs = [synth.activations(Cc, tokens, seed + j) for j in range(len(rows))]
    dxs = [pkg.lib.DeviceBuffer.from_host(x) for x in xs]
    dys = [pkg.lib.DeviceBuffer(tokens * R * 4, fill=0xFF) for R in rows]
    jobs = (pkg.lib.Q4Job * len(rows))()
    for j, R in enumerate(rows):
        dv, ds, db = dev[j % len(dev)]
        jobs[j] = pkg.lib.Q4Job(dv.ptr, ds.ptr, db.ptr, dxs[j].ptr, dys[j].ptr, R)
    stream = lib.salt_mi355_stream()
    pkg.lib.check(lib.salt_mi355_q4_jobs_t_dev(jobs, len(rows), Cc, tokens, stream), "q4_jobs_t_dev")
    pkg.lib.check(lib.salt_mi355_stream_sync(stream), "sync")
    name = lib.salt_mi355_last_kernel().decode()
    return name, [(weights[j % len(weights)], R, xs[j], dys[j].to_host(np.float32).reshape(tokens, R))
                  for j, R in enumerate(rows)]


# (columns, tokens, rows per job, jobs) -> the launch shape it must take.  Between them the cases reach every entry
# of the 32-row kernel's candidate list, every cut of the rows (1, 2, 4, 8 parts), both register widths, and the
# sixteen-row kernel at eight and at twelve waves, in one pass and in several.
SHAPE_CASES = [
    (2816, 1, 2816, 12, "q4_dot_kernel<1,4,2,16,0> ksplit 1"),
    (2816, 1, 2816, 6, "q4_dot_kernel<1,4,2,16,0> ksplit 2"),
    (2816, 1, 2816, 1, "q4_dot_kernel<1,4,2,16,0> ksplit 4"),
    (4096, 1, 4096, 8, "q4_dot_kernel<1,3,2,16,0> ksplit 1"),
    (4096, 1, 4096, 1, "q4_dot_kernel<1,8,2,16,0> ksplit 8"),
    (8192, 1, 2816, 12, "q4_dot_kernel<1,7,2,32,0> ksplit 1"),
    (8192, 1, 2816, 6, "q4_dot_kernel<1,6,2,16,0> ksplit 2"),
    (8192, 1, 2816, 3, "q4_dot_kernel<1,4,3,16,0> ksplit 4"),
    (8192, 2, 2816, 12, "q4_dot_kernel<2,4,2,32,0> ksplit 1"),
    (4096, 4, 4096, 16, "q4_dot16_kernel<4,8,16>"),
    (2816, 1, 2816, 24, "q4_dot16_kernel<1,8,16>"),
    (2816, 2, 2816, 24, "q4_dot16_kernel<2,12,16>"),
    (8192, 1, 2816, 24, "q4_dot16_kernel<1,12,32>"),
    (8192, 4, 2816, 24, "q4_dot16_kernel<4,8,32> in 2 windows"),    # rows too wide for four tokens' planes at once
    (8192, 3, 2816, 24, "q4_dot16_kernel<3,8,32> in 2 windows"),
    (6272, 4, 2816, 24, "q4_dot16_kernel<4,8,32> in 2 windows"),    # 98 groups: the second window ends inside the row
    (8192, 7, 2816, 24, "q4_dot16_kernel<3,8,32> in 2 windows"),   # four tokens, then three
    (8192, 5, 2800, 24, "q4_dot16_kernel<1,12,32>"),                # four tokens in windows, then one; a ragged last block
    (2816, 7, 2816, 24, "q4_dot16_kernel<4,12,16> x 2 passes"),     # more tokens than one pass holds: one launch
    (2112, 1, 2816, 2, "q4_dot_kernel<1,4,2,16,0> ksplit 4"),     # 33 groups: a step that straddles the row's end
    (6272, 3, 96, 1, None),                                          # 98 groups, three tokens, rows cut in 8
]


@pytest.mark.parametrize("Cc,tokens,R,njobs,kernel", SHAPE_CASES)
def test_every_launch_shape(pkg, oracle, Cc, tokens, R, njobs, kernel):
    print(f"class T shape C={Cc} tokens={tokens} R={R} jobs={njobs}", flush=True)
    weights = [synth.q4_tensor(R, Cc, 900 + k) for k in range(min(njobs, 2))]
    name, results = run_jobs(pkg, Cc, tokens, [R] * njobs, weights, 950)
    print("  ", name, flush=True)
    if kernel is not None:
        assert name == kernel
    for j in sorted({0, njobs // 2, njobs - 1}):
        (vals, scales, biases), rows, xs, got = results[j]
        check(got, reference(oracle, vals, scales, biases, rows, Cc, xs), vals, scales, biases, rows, Cc, xs)


def test_the_shape_cases_cover_the_candidate_list():
    reached = {k for *_, k in SHAPE_CASES if k}
    for waves, stages in ((4, 2), (3, 2), (8, 2), (7, 2), (6, 2), (4, 3)):
        assert any(k.startswith("q4_dot_kernel<") and k.split("<")[1].split(",")[1:3] == [str(waves), str(stages)]
                   for k in reached), (waves, stages)
    for cut in (1, 2, 4, 8):
        assert any(k.endswith(f"ksplit {cut}") for k in reached)
    assert any(",32,0>" in k for k in reached) and any("passes" in k for k in reached)
    assert any("<3,8,32> in 2 windows" in k for k in reached) and any("<4,8,32> in 2 windows" in k for k in reached)


def test_same_launch_gives_the_same_bits(pkg):
    """The bits of a tolerance-class result depend on the launch (columns, tokens, number of blocks: they choose the
    kernel shape and with it the order of the fp32 sums) but not on the run: no atomics, no order between
    workgroups.  The same launch, repeated with other launches in between, returns identical bits."""
    for Cc, tokens, R, njobs in ((2816, 1, 2816, 24), (4096, 1, 4096, 1), (8192, 2, 704, 5), (2816, 3, 16384, 1)):
        weights = [synth.q4_tensor(R, Cc, 31)]
        first = run_jobs(pkg, Cc, tokens, [R] * njobs, weights, 40)
        run_jobs(pkg, 1024, 2, [100, 33], [synth.q4_tensor(100, 1024, 32)], 41)
        again = run_jobs(pkg, Cc, tokens, [R] * njobs, weights, 40)
        assert first[0] == again[0]
        for (_, _, _, a), (_, _, _, b) in zip(first[1], again[1]):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
