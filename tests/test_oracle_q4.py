"""Pins the affine-Q4 part of the CPU checker.

Known answers are the ones the reference's unit tests hold
(tests/test_kernels.c:357-392, 394-451, 453-521, 523-558); the rest is what
the arithmetic fixes: an independent float32 emulation, exact power-of-two
scaling, row independence, and the reference's own sources when compiled.
"""
import numpy as np
import pytest

from oracle_lib import bits, ptr
from __graft_entry__ import load_package

synth = load_package().synth


def orc_matvec(o, vals, scales, biases, R, C, x):
    y = np.full(R, np.nan, dtype=np.float32)
    assert o.orc_q4_matvec(ptr(vals), ptr(scales), ptr(biases), R, C, ptr(x), ptr(y)) == 0
    return y


def emulate_rows(vals, scales, biases, R, C, x):
    """Independent restatement in numpy float32 (vectorised over rows, strictly
    sequential over columns): 32 chains, mul-add-mul-add, stride-4 fold."""
    f = np.float32
    q = ((vals.reshape(-1)[:, None] >> (4 * np.arange(8, dtype=np.uint32))) & 15).reshape(R, C)
    g = (np.arange(R * C) // 64).reshape(R, C)
    s = synth.bf16_bits_to_f32(scales)[g]
    b = synth.bf16_bits_to_f32(biases)[g] if biases is not None else np.zeros((R, C), f)
    acc = np.zeros((R, 32), f)
    for c in range(C):
        w = (q[:, c].astype(f) * s[:, c]).astype(f)
        w = (w + b[:, c]).astype(f)
        p = (w * f(x[c])).astype(f)
        acc[:, c & 31] = (acc[:, c & 31] + p).astype(f)
    part = np.zeros((R, 4), f)
    for a in range(8):
        part = (part + acc[:, 4 * a:4 * a + 4]).astype(f)
    return ((part[:, 0] + part[:, 2]).astype(f) + (part[:, 1] + part[:, 3]).astype(f)).astype(f)


def test_decode_known_vector_and_group_boundary(oracle):
    # tests/test_kernels.c:357-392: q = k % 16, scale 1 -> value q
    q = (np.arange(64) % 16).astype(np.uint8)
    vals = synth.pack_nibbles_u32(q)
    out = np.zeros(64, np.float32)
    oracle.orc_q4_decode(ptr(vals), ptr(np.array([0x3F80], np.uint16)),
                         ptr(np.array([0], np.uint16)), 64, ptr(out))
    assert np.array_equal(out, q.astype(np.float32))
    v2 = np.zeros(9, np.uint32); v2[8] = 5
    out2 = np.zeros(72, np.float32)
    oracle.orc_q4_decode(ptr(v2), ptr(np.array([0x3F80, 0x4000], np.uint16)),
                         ptr(np.zeros(2, np.uint16)), 72, ptr(out2))
    assert out2[64] == 10.0 and not out2[:64].any()


def test_word_map_known_answer_120(oracle):
    # tests/test_kernels.c:453-478
    vals = np.array([0x11111111, 0x22222222, 0x44444444, 0x88888888], np.uint32)
    y = orc_matvec(oracle, vals, np.array([0x3F80], np.uint16), np.array([0], np.uint16),
                   1, 32, np.ones(32, np.float32))
    assert y[0] == 120.0


def test_unaligned_sources_known_answer_64(oracle):
    # tests/test_kernels.c:480-521: every pointer sits on an odd byte
    raw_v = np.zeros(40, np.uint8); raw_s = np.zeros(4, np.uint8); raw_b = np.zeros(4, np.uint8)
    ov = (1 - raw_v.ctypes.data) % 4
    os_ = (1 - raw_s.ctypes.data) % 2
    ob = (1 - raw_b.ctypes.data) % 2
    raw_v[ov:ov + 32] = np.tile(np.frombuffer(np.uint32(0x11111111).tobytes(), np.uint8), 8)
    raw_s[os_:os_ + 2] = np.frombuffer(np.uint16(0x3F80).tobytes(), np.uint8)
    import ctypes as C
    y = np.zeros(1, np.float32)
    x = np.ones(64, np.float32)
    rc = oracle.orc_q4_matvec(C.c_void_p(raw_v.ctypes.data + ov), C.c_void_p(raw_s.ctypes.data + os_),
                              C.c_void_p(raw_b.ctypes.data + ob), 1, 64, ptr(x), ptr(y))
    assert rc == 0 and y[0] == 64.0


def test_c8192_all_ones_vs_emulation(oracle):
    # tests/test_kernels.c:523-558
    R, C = 2, 8192
    vals = np.full(R * C // 8, 0x11111111, np.uint32)
    scales = np.full(R * C // 64, 0x3F80, np.uint16)
    biases = np.zeros(R * C // 64, np.uint16)
    x = (((np.arange(C) * 11) % 29 - 14).astype(np.float32) * np.float32(0.001)).astype(np.float32)
    y = orc_matvec(oracle, vals, scales, biases, R, C, x)
    assert np.array_equal(bits(y), bits(emulate_rows(vals, scales, biases, R, C, x)))
    assert np.allclose(y, x.astype(np.float64).sum(), rtol=1e-5, atol=1e-5)


def test_general_shape_vs_naive_sequential(oracle):
    # tests/test_kernels.c:394-451: R=8, C=200 (not a multiple of 64) within 1e-3
    R, C = 8, 200
    g = synth.rng(13)
    q = g.integers(0, 16, size=R * C, dtype=np.uint8)
    vals = synth.pack_nibbles_u32(q)
    ng = (R * C + 63) // 64
    scales = g.integers(0, 20000, size=ng).astype(np.uint16)
    biases = g.integers(0, 20000, size=ng).astype(np.uint16)
    x = (g.integers(0, 200, size=C) / 100.0 - 1.0).astype(np.float32)
    y = orc_matvec(oracle, vals, scales, biases, R, C, x)
    k = np.arange(R * C)
    w = q.astype(np.float64) * synth.bf16_bits_to_f32(scales)[k // 64] + synth.bf16_bits_to_f32(biases)[k // 64]
    naive = (w.reshape(R, C) * x[None, :]).sum(axis=1)
    assert np.all(np.abs(y - naive) <= 1e-3 * (1 + np.abs(naive)))
    assert np.array_equal(bits(y), bits(emulate_rows(vals, scales, biases, R, C, x)))


@pytest.mark.parametrize("R,C,seed", [(5, 64, 1), (3, 704, 2), (4, 2816, 3), (7, 96, 4)])
def test_matches_independent_emulation(oracle, R, C, seed):
    pad = (-(R * C)) % 64
    vals, scales, biases = synth.q4_tensor(1, R * C + pad, seed)
    x = synth.activations(C, 1, seed + 100)[0]
    y = orc_matvec(oracle, vals, scales, biases, R, C, x)
    assert np.array_equal(bits(y), bits(emulate_rows(vals[:R * C // 8], scales, biases, R, C, x)))


def test_power_of_two_scaling_is_exact_and_rows_are_independent(oracle):
    R, C = 16, 512
    vals, scales, biases = synth.q4_tensor(R, C, 7)
    x = synth.activations(C, 1, 8)[0]
    y = orc_matvec(oracle, vals, scales, biases, R, C, x)
    y8 = orc_matvec(oracle, vals, scales, biases, R, C, (x * np.float32(8)).astype(np.float32))
    assert np.array_equal(bits(y8), bits(y * np.float32(8)))
    assert not orc_matvec(oracle, vals, scales, biases, R, C, np.zeros(C, np.float32)).view(np.uint32).any()
    # rows r0..r1 alone give the same bits as the full call
    part = np.zeros(R, np.float32)
    assert oracle.orc_q4_matvec_rows(ptr(vals), ptr(scales), ptr(biases), R, C, ptr(x), ptr(part), 5, 9) == 0
    assert np.array_equal(bits(part[5:9]), bits(y[5:9])) and not part[:5].any() and not part[9:].any()
    # a row's result does not depend on the other rows' weights
    vals2 = vals.copy(); vals2[:C // 8 * 3] ^= 0x5A5A5A5A
    y2 = orc_matvec(oracle, vals2, scales, biases, R, C, x)
    assert np.array_equal(bits(y2[3:]), bits(y[3:]))


def test_batch_and_threads_equal_single_calls(oracle):
    R, C, B = 2048 + 32, 128, 3
    vals, scales, biases = synth.q4_tensor(R, C, 11)
    xs = synth.activations(C, B, 12)
    ys = np.zeros((B, R), np.float32)
    assert oracle.orc_q4_matvec_batch(ptr(vals), ptr(scales), ptr(biases), R, C, B, ptr(xs), ptr(ys)) == 0
    for t in range(B):
        assert np.array_equal(bits(ys[t]), bits(orc_matvec(oracle, vals, scales, biases, R, C, xs[t])))
    yt = np.zeros(R, np.float32)
    assert oracle.orc_q4_matvec_threads(ptr(vals), ptr(scales), ptr(biases), R, C, ptr(xs[0]), ptr(yt), 5) == 0
    assert np.array_equal(bits(yt), bits(ys[0]))


def test_rejects_bad_arguments(oracle):
    v = np.zeros(8, np.uint32); s = np.zeros(1, np.uint16); x = np.zeros(64, np.float32); y = np.zeros(1, np.float32)
    assert oracle.orc_q4_matvec(None, ptr(s), ptr(s), 1, 64, ptr(x), ptr(y)) == -1
    assert oracle.orc_q4_matvec(ptr(v), ptr(s), ptr(s), 0, 64, ptr(x), ptr(y)) == -1
    assert oracle.orc_q4_matvec(ptr(v), ptr(s), ptr(s), 1, 0, ptr(x), ptr(y)) == -1
    # biases may be NULL: bias 0 (reference src/kernels.c:232-233)
    v[:] = 0x11111111; s[0] = 0x3F80; x[:] = 1
    assert oracle.orc_q4_matvec(ptr(v), ptr(s), None, 1, 64, ptr(x), ptr(y)) == 0 and y[0] == 64.0


# ---- against the reference's own sources, when they have been compiled ----

@pytest.mark.parametrize("R,C", [(704, 2816), (705, 2816), (2048, 2816), (64, 8192), (2816, 704), (9, 200), (3, 8256)])
@pytest.mark.parametrize("simd", [0, 1])
def test_equals_compiled_reference(oracle, reference, R, C, simd):
    pad = (-(R * C)) % 64
    vals, scales, biases = synth.q4_tensor(1, R * C + pad, R * 7 + C)
    vals = np.concatenate([vals, np.zeros(8, np.uint32)])
    x = synth.activations(C, 1, 5)[0]
    want = np.zeros(R, np.float32)
    reference.salt_kernels_set_simd(simd)
    try:
        if simd and C % 16:
            pytest.skip("reference SIMD tail differs from its canonical row when C % 16 != 0")
        assert reference.salt_q4_matvec_status(ptr(vals), ptr(scales), ptr(biases), R, C, ptr(x), ptr(want)) == 0
    finally:
        reference.salt_kernels_set_simd(1)
    got = orc_matvec(oracle, vals, scales, biases, R, C, x)
    assert np.array_equal(bits(got), bits(want))


def test_decode_equals_compiled_reference(oracle, reference):
    n = 64 * 37
    vals, scales, biases = synth.q4_tensor(1, n, 99)
    a = np.zeros(n, np.float32); b = np.zeros(n, np.float32)
    oracle.orc_q4_decode(ptr(vals), ptr(scales), ptr(biases), n, ptr(a))
    reference.salt_q4_decode(ptr(vals), ptr(scales), ptr(biases), n, ptr(b))
    assert np.array_equal(bits(a), bits(b))


def test_batch_equals_compiled_reference(oracle, reference):
    R, C, B = 705, 2816, 3
    pad = (-(R * C)) % 64
    vals, scales, biases = synth.q4_tensor(1, R * C + pad, 21)
    xs = synth.activations(C, B, 22)
    got = np.zeros((B, R), np.float32); want = np.zeros((B, R), np.float32)
    assert oracle.orc_q4_matvec_batch(ptr(vals), ptr(scales), ptr(biases), R, C, B, ptr(xs), ptr(got)) == 0
    assert reference.salt_q4_matvec_batch_rows(ptr(vals), ptr(scales), ptr(biases), R, C, B, ptr(xs), ptr(want), 0, R) == 0
    assert np.array_equal(bits(got), bits(want))
