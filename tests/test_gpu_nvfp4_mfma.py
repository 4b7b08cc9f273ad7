"""Prefill-sized NVFP4 matmul on the matrix cores: tolerance class.

Both operands reach the matrix cores as exact bf16 values (code * block scale),
so the result differs from the reference matvec (src/nvfp4.c:228-256) only by
the order of the fp32 additions and by where the two per-tensor factors are
rounded.  Stated tolerance per output, checked against the bit-exact CPU
checker:

    |error| <= 2^-20 * sum_c |w_c * x_c| + 1e-30

with w_c, x_c the reference's dequantised weight and activation."""
import ctypes as C

import numpy as np
import pytest

from golden import cases
from oracle_lib import ptr

pytestmark = pytest.mark.gpu
synth = cases.synth


def reference(oracle, packed, scales, divisor, g, R, Cc, xs):
    B = xs.shape[0]
    want = np.zeros((B, R), np.float32)
    xdq = np.zeros((B, Cc), np.float32)
    for t in range(B):
        xp = np.zeros(Cc // 2, np.uint8); xsb = np.zeros(Cc // 16, np.uint8)
        assert oracle.orc_nvfp4_matvec(ptr(packed), ptr(scales), divisor, g, R, Cc, ptr(xs[t]), ptr(want[t]),
                                       ptr(xp), ptr(xsb), ptr(xdq[t])) == 0
    wdq = np.zeros(R * Cc, np.float32)
    assert oracle.orc_nvfp4_dequant_weights(ptr(packed), ptr(scales), divisor, R, Cc, ptr(wdq)) == 0
    return want, np.abs(xdq.astype(np.float64)) @ np.abs(wdq.reshape(R, Cc).astype(np.float64)).T


@pytest.mark.parametrize("R,Cc,B,g", [(128, 64, 128, 64.0), (192, 256, 37, 8.0), (70, 128, 1, 64.0),
                                      (512, 2048, 256, 100.0), (1000, 1024, 130, 1.0),
                                      (295, 1920, 191, 17.5)])     # 30 column chunks over 6 tiles: an uneven split of K
def test_matmul_within_stated_tolerance(pkg, oracle, R, Cc, B, g):
    print(f"nvfp4 mfma R={R} C={Cc} B={B}", flush=True)
    packed, scales = synth.nvfp4_tensor(R, Cc, R + Cc + B)
    divisor = 1234.5
    xs = synth.activations(Cc, B, 5)
    xs[0, :4] = [0.0, -0.0, 1e-20, 40.0]
    status, got = pkg.lib.nvfp4_matmul(packed, scales, divisor, g, R, Cc, xs)
    assert status == 0
    want, mags = reference(oracle, packed, scales, divisor, g, R, Cc, xs)
    bound = 2.0 ** -20 * mags + 1e-30
    err = np.abs(got.astype(np.float64) - want)
    ratio = float((err / bound).max())
    print("max err / bound", ratio, flush=True)
    assert np.isfinite(got).all() and ratio <= 1.0, ratio


def test_cfg4_8192x8192_batch256_sampled_rows(pkg, oracle):
    """BASELINE configs[4] at batch 256 and full size (128 tiles x 4 K-splits plus the split sum): 32 rows x 256
    tokens against the checker."""
    R = Cc = 8192
    B = 256
    print("nvfp4 mfma 8192 x 8192 x 256", flush=True)
    packed, scales = synth.nvfp4_tensor(R, Cc, 40)
    xs = synth.activations(Cc, B, 42)
    status, got = pkg.lib.nvfp4_matmul(packed, scales, 2688.0, 64.0, R, Cc, xs)
    assert status == 0 and np.isfinite(got).all()
    rows = np.arange(5, R, 256)
    sub_packed = np.ascontiguousarray(packed.reshape(R, Cc // 2)[rows]).reshape(-1)
    sub_scales = np.ascontiguousarray(scales.reshape(R, Cc // 16)[rows]).reshape(-1)
    want, mags = reference(oracle, sub_packed, sub_scales, 2688.0, 64.0, len(rows), Cc, xs)
    bound = 2.0 ** -20 * mags + 1e-30
    err = np.abs(got[:, rows].astype(np.float64) - want)
    ratio = float((err / bound).max())
    print("max err / bound", ratio, flush=True)
    assert ratio <= 1.0, ratio


def test_non_finite_activation_publishes_nothing(pkg):
    R, Cc, B = 128, 128, 9
    packed, scales = synth.nvfp4_tensor(R, Cc, 3)
    xs = synth.activations(Cc, B, 4)
    xs[5, 77] = np.inf
    status, got = pkg.lib.nvfp4_matmul(packed, scales, 2.0, 64.0, R, Cc, xs)
    assert status == -1 and (got.view(np.uint32) == 0xFFFFFFFF).all()
    xs[5, 77] = np.nan
    status, got = pkg.lib.nvfp4_matmul(packed, scales, 2.0, 64.0, R, Cc, xs)
    assert status == -1 and (got.view(np.uint32) == 0xFFFFFFFF).all()
    lib = pkg.lib.init()
    assert lib.salt_mi355_nvfp4_matmul_dev(None, None, 2.0, 64.0, R, Cc, B, None, None, None, None, None) == -1
    assert lib.salt_mi355_nvfp4_matmul_workspace_bytes(R, 96, B) == 0      # C must be a multiple of 64
