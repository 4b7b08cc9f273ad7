"""CPU checker for the bf16 matvec (LM head) and the 8-bit affine matvec
(router gates): pinned by the reference's own compiled functions (both its
scalar and its SIMD realisation), by closed forms, and by an independent
float32 emulation."""
import numpy as np
import pytest

from golden import cases
from oracle_lib import bits, ptr

synth = cases.synth


def bf16_matrix(R, C, seed):
    return (synth.rng(seed).standard_normal(R * C).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)


def emulate_bf16_row(row, x, bias):
    f = np.float32
    w = (row.astype(np.uint32) << 16).view(np.float32)
    a = [f(0)] * 8
    C = len(row)
    c = 0
    while c + 7 < C:
        for j in range(8):
            a[j] = f(a[j] + f(w[c + j] * x[c + j]))
        c += 8
    s = f(f(f(a[0] + a[2]) + f(a[4] + a[6])) + f(f(a[1] + a[3]) + f(a[5] + a[7])))
    while c < C:
        s = f(s + f(w[c] * x[c]))
        c += 1
    return f(s + (bias if bias is not None else f(0)))


@pytest.mark.parametrize("R,C", [(1, 8), (3, 16), (6, 150), (5, 7), (4, 2816), (2, 33)])
def test_bf16_matvec_emulation_and_closed_forms(oracle, R, C):
    W = bf16_matrix(R, C, R * 100 + C)
    x = synth.activations(C, 1, C + 3)[0]
    bias = synth.activations(R, 1, 9)[0]
    y = np.zeros(R, np.float32)
    oracle.orc_bf16_matvec(ptr(W), R, C, ptr(x), ptr(bias), ptr(y))
    for r in range(R):
        assert bits(np.float32(y[r])) == bits(emulate_bf16_row(W[r * C:(r + 1) * C], x, bias[r]))
    oracle.orc_bf16_matvec(ptr(W), R, C, ptr(x), None, ptr(y))
    for r in range(R):
        assert bits(np.float32(y[r])) == bits(emulate_bf16_row(W[r * C:(r + 1) * C], x, None))
    ones = np.full(R * C, 0x3F80, np.uint16)                   # 1.0
    oracle.orc_bf16_matvec(ptr(ones), R, C, ptr(np.ones(C, np.float32)), None, ptr(y))
    assert (y == C).all()
    # a dropped chain, a wrong fold or a transposed operand changes this: x = column index, W = 2^(c % 8)
    powers = np.tile((np.float32(2.0) ** (np.arange(C) % 8)).astype(np.float32).view(np.uint32) >> 16, R).astype(np.uint16)
    xi = np.arange(C, dtype=np.float32)
    oracle.orc_bf16_matvec(ptr(powers), R, C, ptr(xi), None, ptr(y))
    assert (y == float(np.sum((2.0 ** (np.arange(C) % 8)) * np.arange(C)))).all()       # exact in fp32 at these sizes


@pytest.mark.parametrize("R,C", [(6, 150), (8, 2816), (3, 64), (2, 8200)])
def test_bf16_matvec_equals_compiled_reference(oracle, reference, R, C):
    W = bf16_matrix(R, C, R + C)
    # the reference's own test pattern as well (tests/test_kernels.c:226-238); half of its weights are NaN
    # encodings, so its rows are NaN and only that is compared there (NaN payloads are not part of the contract)
    if (R, C) == (6, 150):
        W = np.array([((i * 7 % 200) - 100) & 0xFFFF for i in range(R * C)], np.uint16)
    x = synth.activations(C, 1, 5)[0]
    if (R, C) == (6, 150):
        x = (((np.arange(C) % 6) - 3) * np.float32(0.2)).astype(np.float32)
    bias = synth.activations(R, 1, 6)[0]
    want = np.zeros(R, np.float32); got = np.zeros(R, np.float32)
    for use_bias in (None, bias):
        b = ptr(use_bias) if use_bias is not None else None
        oracle.orc_bf16_matvec(ptr(W), R, C, ptr(x), b, ptr(got))
        for simd in (0, 1):
            reference.salt_kernels_set_simd(simd)
            reference.salt_bf16_matvec(ptr(W), R, C, ptr(x), b, ptr(want))
            assert np.array_equal(np.isnan(got), np.isnan(want))
            ok = ~np.isnan(want)
            assert np.array_equal(bits(got)[ok], bits(want)[ok]), (simd, use_bias is not None)
            assert ok.all() or (R, C) == (6, 150)
    reference.salt_kernels_set_simd(1)


def q8_tensor(R, C, seed):
    g = synth.rng(seed)
    vals = g.integers(0, 256, size=R * C, dtype=np.uint8)
    groups = (R * C + 63) // 64
    scales = (g.uniform(0.001, 0.01, groups).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    biases = (g.uniform(-1.0, 0.0, groups).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    return vals, scales, biases


@pytest.mark.parametrize("R,C", [(1, 64), (4, 128), (128, 2816), (3, 96)])
def test_q8_matvec_pins(oracle, reference, R, C):
    vals, scales, biases = q8_tensor(R, C, R * 3 + C)
    x = synth.activations(C, 1, 12)[0]
    got = np.zeros(R, np.float32); want = np.zeros(R, np.float32)
    for b in (biases, None):
        bp = ptr(b) if b is not None else None
        oracle.orc_q8_matvec(ptr(vals), ptr(scales), bp, R, C, ptr(x), ptr(got))
        reference.salt_q8_matvec(ptr(vals), ptr(scales), bp, R, C, ptr(x), ptr(want))
        assert np.array_equal(bits(got), bits(want))
    # closed form: scale 1, bias 0, x = 1 -> the sum of the bytes, exact
    one = np.full(scales.size, 0x3F80, np.uint16)
    oracle.orc_q8_matvec(ptr(vals), ptr(one), None, R, C, ptr(np.ones(C, np.float32)), ptr(got))
    assert np.array_equal(got, vals.reshape(R, C).astype(np.float64).sum(axis=1).astype(np.float32))
    # serial order: a single chain, so a huge then tiny sequence keeps the textbook left-to-right result
    f = np.float32
    row = np.zeros(C, np.float32); row[0] = 3e7; row[1:] = 1.0
    oracle.orc_q8_matvec(ptr(np.ones(R * C, np.uint8)), ptr(one), None, R, C, ptr(row), ptr(got))
    acc = f(0)
    for v in row:
        acc = f(acc + v)
    assert (got == acc).all()
