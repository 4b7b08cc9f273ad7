"""Tolerance-class NVFP4 reference matvec (salt_mi355_nvfp4_matvec_t_dev, salt_mi355_nvfp4_jobs_t_dev).

The kernel quantises the activation exactly as the reference does (same codes, same block scales), adds the code
products of every 16-column block exactly and applies the block's two factors once; only the order and the rounding
of the fp32 sum over the blocks differ from the reference matvec (src/nvfp4.c:228-256).  Stated tolerance per output,
checked against the bit-exact CPU checker:

    |error| <= 2^-20 * sum_c |w_c * x_c| + 1e-30

with w_c, x_c the reference's dequantised weight and activation."""
import numpy as np
import pytest

from golden import cases
from oracle_lib import ptr

pytestmark = pytest.mark.gpu
synth = cases.synth


def reference(oracle, packed, scales, divisor, g, R, Cc, xs, rows=None):
    """Reference outputs and sum_c |w x| for the listed rows (all when None)."""
    rows = np.arange(R) if rows is None else np.asarray(rows)
    sub_packed = np.ascontiguousarray(packed.reshape(R, Cc // 2)[rows]).reshape(-1)
    sub_scales = np.ascontiguousarray(scales.reshape(R, Cc // 16)[rows]).reshape(-1)
    n = len(rows)
    B = xs.shape[0]
    want = np.zeros((B, n), np.float32)
    xdq = np.zeros((B, Cc), np.float32)
    for t in range(B):
        xp = np.zeros(Cc // 2, np.uint8); xsb = np.zeros(Cc // 16, np.uint8)
        assert oracle.orc_nvfp4_matvec(ptr(sub_packed), ptr(sub_scales), divisor, g, n, Cc, ptr(xs[t]), ptr(want[t]),
                                       ptr(xp), ptr(xsb), ptr(xdq[t])) == 0
    wdq = np.zeros(n * Cc, np.float32)
    assert oracle.orc_nvfp4_dequant_weights(ptr(sub_packed), ptr(sub_scales), divisor, n, Cc, ptr(wdq)) == 0
    return want, np.abs(xdq.astype(np.float64)) @ np.abs(wdq.reshape(n, Cc).astype(np.float64)).T


def check(got, want, mags):
    bound = 2.0 ** -20 * mags + 1e-30
    err = np.abs(got.astype(np.float64) - want)
    ratio = float((err / bound).max())
    print("max err / bound", ratio, flush=True)
    assert np.isfinite(got).all() and ratio <= 1.0, ratio


@pytest.mark.parametrize("R,Cc,B,g", [
    (96, 2816, 1, 64.0), (257, 512, 3, 8.0), (33, 576, 2, 1.0), (1, 1024, 1, 100.0), (300, 4096, 4, 17.5),
    (64, 8192, 5, 64.0), (2816, 704, 1, 64.0),
    (70, 128, 2, 64.0), (40, 96, 1, 64.0),             # below 512 columns / not a multiple of 64: the bit-exact kernel
])
def test_matvec_within_stated_tolerance(pkg, oracle, R, Cc, B, g):
    print(f"nvfp4 class T R={R} C={Cc} B={B}", flush=True)
    packed, scales = synth.nvfp4_tensor(R, Cc, R + Cc + B)
    xs = synth.activations(Cc, B, 5)
    xs[0, :4] = [0.0, -0.0, 1e-20, 40.0]
    status, got = pkg.lib.nvfp4_matvec_t(packed, scales, 1234.5, R, Cc, xs, g)
    assert status == 0
    want, mags = reference(oracle, packed, scales, 1234.5, g, R, Cc, xs)
    check(got, want, mags)


def test_cfg4_8192x8192_batch1_sampled_rows(pkg, oracle):
    """BASELINE configs[4] at its full size: every 37th row against the checker (the scalar reference row costs
    ~0.1 ms per row and token)."""
    R = Cc = 8192
    packed, scales = synth.nvfp4_tensor(R, Cc, 40)
    xs = synth.activations(Cc, 1, 541)
    status, got = pkg.lib.nvfp4_matvec_t(packed, scales, 2688.0, R, Cc, xs, 64.0)
    assert status == 0 and np.isfinite(got).all()
    rows = np.arange(0, R, 37)
    want, mags = reference(oracle, packed, scales, 2688.0, 64.0, R, Cc, xs, rows)
    check(got[:, rows], want, mags)


def test_nan_scale_codes_and_negative_divisor(pkg, oracle):
    R, Cc = 64, 1024
    packed, scales = synth.nvfp4_tensor(R, Cc, 9)
    scales = scales.copy()
    scales.reshape(R, Cc // 16)[5, 3] = 0x7F                    # NaN block scale: that row is NaN, as in the reference
    scales.reshape(R, Cc // 16)[9, 60] = 0xFF
    xs = synth.activations(Cc, 2, 10)
    status, got = pkg.lib.nvfp4_matvec_t(packed, scales, -3.0, R, Cc, xs, 64.0)
    want, mags = reference(oracle, packed, scales, -3.0, 64.0, R, Cc, xs)
    assert status == 0
    assert np.isnan(got[:, [5, 9]]).all() and np.isnan(want[:, [5, 9]]).all()
    keep = [r for r in range(R) if r not in (5, 9)]
    check(got[:, keep], want[:, keep], mags[:, keep])


def test_non_finite_activation_publishes_nothing(pkg):
    R, Cc, B = 128, 1024, 3
    packed, scales = synth.nvfp4_tensor(R, Cc, 3)
    xs = synth.activations(Cc, B, 4)
    for poison in (np.inf, np.nan):
        xs[1, 777] = poison
        status, got = pkg.lib.nvfp4_matvec_t(packed, scales, 2.0, R, Cc, xs, 64.0)
        assert status == -1 and (got.view(np.uint32) == 0xFFFFFFFF).all()
    lib = pkg.lib.init()
    buf = pkg.lib.DeviceBuffer(1 << 14)
    assert lib.salt_mi355_nvfp4_matvec_t_dev(buf.ptr, buf.ptr, 2.0, 64.0, 8, 1024, 1, buf.ptr, buf.ptr, None, None) == -1
    assert lib.salt_mi355_nvfp4_matvec_t_dev(buf.ptr, buf.ptr, 0.0, 64.0, 8, 1024, 1, buf.ptr, buf.ptr, buf.ptr, None) == -1


def test_many_jobs_one_launch(pkg, oracle):
    lib = pkg.lib.init()
    Cc, tokens, g = 2048, 2, 64.0
    rows = [300, 33, 1024, 1]
    held, jobs, expect = [], (pkg.lib.Fp4Job * len(rows))(), []
    for j, R in enumerate(rows):
        packed, scales = synth.nvfp4_tensor(R, Cc, 100 + j)
        xs = synth.activations(Cc, tokens, 200 + j)
        dw, ds, dx = (pkg.lib.DeviceBuffer.from_host(a) for a in (packed, scales, xs))
        dy = pkg.lib.DeviceBuffer(tokens * R * 4, fill=0xFF)
        held.append((dw, ds, dx, dy))
        jobs[j] = pkg.lib.Fp4Job(dw.ptr, ds.ptr, 7.0 + j, dx.ptr, dy.ptr, R)
        expect.append((packed, scales, 7.0 + j, R, xs))
    status = pkg.lib.DeviceBuffer(4, fill=0)
    stream = lib.salt_mi355_stream()
    pkg.lib.check(lib.salt_mi355_nvfp4_jobs_t_dev(jobs, len(rows), Cc, tokens, g, status.ptr, stream), "nvfp4_jobs_t_dev")
    pkg.lib.check(lib.salt_mi355_stream_sync(stream), "sync")
    assert int(status.to_host(np.int32)[0]) == 0
    for (dw, ds, dx, dy), (packed, scales, divisor, R, xs) in zip(held, expect):
        got = dy.to_host(np.float32).reshape(tokens, R)
        want, mags = reference(oracle, packed, scales, divisor, g, R, Cc, xs)
        check(got, want, mags)
