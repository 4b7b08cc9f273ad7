"""bf16 (language-model head) and 8-bit affine (router gate) matvecs on the MI355X through the C ABI, bit-for-bit
against the CPU checker."""
import numpy as np
import pytest

from golden import cases
from oracle_lib import bits, ptr

pytestmark = pytest.mark.gpu
synth = cases.synth


@pytest.fixture(scope="module")
def gpu(pkg):
    pkg.lib.init()
    return pkg.lib


def bf16_matrix(R, C, seed):
    return (synth.rng(seed).standard_normal(R * C).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)


def oracle_bf16(oracle, W, R, C, xs, bias):
    out = np.zeros((xs.shape[0], R), np.float32)
    for t in range(xs.shape[0]):
        oracle.orc_bf16_matvec(ptr(W), R, C, ptr(np.ascontiguousarray(xs[t])), ptr(bias) if bias is not None else None,
                               ptr(out[t]))
    return out


# streaming kernel: full chunks, a partial last chunk, ragged row tiles, one to five activation rows
@pytest.mark.parametrize("R,C,B", [(64, 64, 1), (200, 2816, 1), (1000, 8, 1), (77, 200, 2), (129, 1096, 3),
                                   (4096, 2816, 4), (65, 72, 5), (3, 8192, 1), (8192, 512, 1)])
def test_bf16_matvec_streaming(gpu, oracle, R, C, B):
    print("bf16 stream", R, C, B, flush=True)
    W = bf16_matrix(R, C, R + C)
    xs = synth.activations(C, B, R * 7 + B)
    bias = synth.activations(R, 1, 4)[0]
    for b in (None, bias):
        got = gpu.bf16_matvec(W, R, C, xs, b)
        want = oracle_bf16(oracle, W, R, C, xs, b)
        assert np.array_equal(bits(got), bits(want)), (R, C, B, b is not None)


# any column count, any weight address: the per-row kernel, with the scalar tail past the last multiple of eight
@pytest.mark.parametrize("R,C,B,offset", [(6, 150, 1, 0), (70, 7, 2, 0), (33, 264, 1, 2), (130, 96, 3, 6), (5, 1, 1, 0)])
def test_bf16_matvec_any_shape(gpu, oracle, R, C, B, offset):
    print("bf16 generic", R, C, B, offset, flush=True)
    W = bf16_matrix(R, C, R * 3 + C)
    xs = synth.activations(C, B, 11)
    got = gpu.bf16_matvec(W, R, C, xs, None, weight_offset=offset)
    assert np.array_equal(bits(got), bits(oracle_bf16(oracle, W, R, C, xs, None)))


def test_bf16_matvec_signed_zero_and_subnormals(gpu, oracle):
    print("bf16 zero", flush=True)
    R, C = 64, 64
    W = np.full(R * C, 0x8000, np.uint16)                       # -0.0 everywhere: the result is +0.0 (s + 0.0f)
    x = np.ones((1, C), np.float32)
    got = gpu.bf16_matvec(W, R, C, x)
    assert (bits(got) == 0).all()
    W = np.full(R * C, 0x0001, np.uint16)                       # bf16 subnormal weights survive
    got = gpu.bf16_matvec(W, R, C, x)
    assert np.array_equal(bits(got), bits(oracle_bf16(oracle, W, R, C, x, None))) and (got != 0).all()


def test_bf16_matvec_head_shape(gpu, oracle):
    """Rows of a full-width head tile (2816 columns) against the checker on a row sample, and linearity in the bias
    over every row."""
    print("bf16 head", flush=True)
    R, C = 32768, 2816
    W = bf16_matrix(R, C, 99)
    x = synth.activations(C, 1, 17)
    got = gpu.bf16_matvec(W, R, C, x)[0]
    sample = np.concatenate([np.arange(0, 128), np.arange(R - 130, R), synth.rng(5).integers(0, R, 256)])
    for r in sample:
        want = np.zeros(1, np.float32)
        oracle.orc_bf16_matvec(ptr(W[r * C:(r + 1) * C].copy()), 1, C, ptr(x[0]), None, ptr(want))
        assert bits(got[r:r + 1])[0] == bits(want)[0], r
    bias = synth.activations(R, 1, 2)[0]
    with_bias = gpu.bf16_matvec(W, R, C, x, bias)[0]
    # y_with_bias = fl(s + bias) and y = fl(s + 0) = s for every row
    assert np.array_equal(bits(with_bias), bits((got + bias).astype(np.float32)))


def q8_tensor(R, C, seed):
    g = synth.rng(seed)
    vals = g.integers(0, 256, size=R * C, dtype=np.uint8)
    groups = (R * C + 63) // 64
    scales = (g.uniform(0.001, 0.01, groups).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    biases = (g.uniform(-1.0, 0.0, groups).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    return vals, scales, biases


@pytest.mark.parametrize("R,C,B,offset", [(128, 2816, 1, 0), (128, 2816, 5, 0), (1, 64, 1, 0), (70, 128, 2, 0),
                                          (3, 96, 2, 0), (65, 200, 1, 0), (16, 256, 1, 4), (20, 384, 1, 0), (17, 576, 3, 0),
                                          (33, 4096, 1, 0), (40, 4160, 2, 0), (130, 1728, 1, 0)])
def test_q8_matvec(gpu, oracle, R, C, B, offset):
    print("q8", R, C, B, offset, flush=True)
    vals, scales, biases = q8_tensor(R, C, R + C)
    xs = synth.activations(C, B, 3)
    for b in (biases, None):
        got = gpu.q8_matvec(vals, scales, b, R, C, xs, value_offset=offset)
        want = np.zeros((B, R), np.float32)
        for t in range(B):
            oracle.orc_q8_matvec(ptr(vals), ptr(scales), ptr(b) if b is not None else None, R, C,
                                 ptr(np.ascontiguousarray(xs[t])), ptr(want[t]))
        assert np.array_equal(bits(got), bits(want)), (R, C, B, b is not None)


def test_argument_errors(gpu):
    lib = gpu.load()
    buf = gpu.DeviceBuffer(4096)
    assert lib.salt_mi355_bf16_matvec_dev(None, 4, 8, 1, buf.ptr, None, buf.ptr, None) == -1
    assert lib.salt_mi355_bf16_matvec_dev(buf.ptr, 0, 8, 1, buf.ptr, None, buf.ptr, None) == -1
    assert lib.salt_mi355_q8_matvec_dev(buf.ptr, None, None, 4, 64, 1, buf.ptr, buf.ptr, None) == -1
    assert lib.salt_mi355_q8_matvec_dev(buf.ptr, buf.ptr, None, 4, 0, 1, buf.ptr, buf.ptr, None) == -1
