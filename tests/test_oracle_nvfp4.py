"""Pins the NVFP4 part of the CPU checker: reference golden bytes and bit
patterns (tests/test_nvfp4.c:28-117), the OCP FP8/FP4 tables as torch decodes
them, closed-form encoders against the argmin scans, and the reference's own
sources when compiled."""
import ctypes as C

import numpy as np
import pytest

from oracle_lib import bits, ptr
from __graft_entry__ import load_package

synth = load_package().synth

# data held by the reference's own test (tests/test_nvfp4.c:57-83)
QDQ_INPUT = np.array([-6.0, -5.0, -4.0, -3.0, -2.0, -1.5, -1.0, -0.5,
                      0.0, 0.25, 0.5, 0.75, 1.0, 2.0, 4.0, 6.0,
                      -3.0, -2.5, -2.0, -1.5, -1.0, -0.5, 0.0, 0.25,
                      0.5, 0.75, 1.0, 1.5, 2.0, 2.5, 3.0, 0.0], np.float32)
QDQ_PACKED = np.array([239, 222, 188, 154, 0, 33, 66, 118, 239, 222, 172, 16, 50, 84, 102, 7], np.uint8)
QDQ_SCALES = np.array([104, 96], np.uint8)
QDQ_DEQUANT_BITS = np.array([
    0xc0c00000, 0xc0800000, 0xc0800000, 0xc0400000, 0xc0000000, 0xbfc00000, 0xbf800000, 0xbf000000,
    0x00000000, 0x00000000, 0x3f000000, 0x3f800000, 0x3f800000, 0x40000000, 0x40800000, 0x40c00000,
    0xc0400000, 0xc0000000, 0xc0000000, 0xbfc00000, 0xbf800000, 0xbf000000, 0x00000000, 0x3e800000,
    0x3f000000, 0x3f400000, 0x3f800000, 0x3fc00000, 0x40000000, 0x40000000, 0x40400000, 0x00000000], np.uint32)


def test_e2m1_codebook(oracle):
    positive = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    for i, v in enumerate(positive):
        assert oracle.orc_e2m1(i) == v
        assert oracle.orc_e2m1(i | 8) == -v
    assert bits(np.float32(oracle.orc_e2m1(8)))[()] == 0  # "-0" decodes to +0


def test_e4m3fn_points_and_torch_table(oracle):
    assert oracle.orc_e4m3fn(0x38) == 1.0 and oracle.orc_e4m3fn(0x68) == 64.0
    assert oracle.orc_e4m3fn(0x7e) == 448.0 and oracle.orc_e4m3fn(0xfe) == -448.0
    assert np.isnan(oracle.orc_e4m3fn(0x7f)) and np.isnan(oracle.orc_e4m3fn(0xff))
    torch = pytest.importorskip("torch")
    table = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    for code in range(256):
        got = oracle.orc_e4m3fn(code)
        assert (np.isnan(got) and np.isnan(table[code])) or got == table[code], code


def test_e4m3fn_encode_points(oracle):
    code = C.c_uint8(0)
    for value, want in [(64.0, 0x68), (448.0, 0x7e), (-448.0, 0xfe), (1e9, 0x7e), (0.0, 0), (-0.0, 0x80)]:
        assert oracle.orc_e4m3fn_encode(value, C.byref(code)) == 0 and code.value == want
    assert oracle.orc_e4m3fn_encode(float("nan"), C.byref(code)) == -1


def _probe_points(grid):
    """Every representable value, every midpoint, and their float32 neighbours."""
    grid = np.asarray(sorted(set(grid)), np.float64)
    mids = (grid[:-1] + grid[1:]) / 2
    pts = np.concatenate([grid, mids]).astype(np.float32)
    pts = np.concatenate([pts, np.nextafter(pts, np.float32(np.inf)), np.nextafter(pts, np.float32(-np.inf))])
    return np.concatenate([pts, -pts])


def test_closed_form_e4m3fn_encoder_equals_scan(oracle):
    grid = [oracle.orc_e4m3fn(c) for c in range(0x7f)]
    pts = np.concatenate([_probe_points(grid),
                          synth.rng(5).uniform(-500, 500, 20000).astype(np.float32),
                          (synth.rng(6).standard_normal(20000) * 0.02).astype(np.float32),
                          np.array([1e-45, 1e-40, 9.7e-4, 9.8e-4, 447.9, 448.1, 1e30, np.inf], np.float32)])
    code = C.c_uint8(0)
    for v in pts:
        assert oracle.orc_e4m3fn_encode(float(v), C.byref(code)) == 0
        assert oracle.orc_e4m3fn_encode_rne(float(v)) == code.value, float(v)


def test_closed_form_e2m1_encoder_equals_scan(oracle):
    pts = np.concatenate([_probe_points([0, .5, 1, 1.5, 2, 3, 4, 6]),
                          synth.rng(7).uniform(-7, 7, 20000).astype(np.float32),
                          np.array([1e-45, 6.5, 100.0, 4096.0], np.float32)])
    # moderate inputs only: the callers clamp to [-6, 6] first; once |v| is so large
    # that float32 cannot tell the distances apart the scan keeps code 0
    for v in pts:
        assert oracle.orc_e2m1_encode_rne(float(v)) == oracle.orc_e2m1_encode(float(v)), float(v)
    assert oracle.orc_e2m1_encode(float("nan")) & 7 == 0 and oracle.orc_e2m1_encode_rne(float("nan")) & 7 == 0


def test_qdq_golden_bytes(oracle):
    packed = np.zeros(16, np.uint8); scales = np.zeros(2, np.uint8); dq = np.zeros(32, np.float32)
    assert oracle.orc_nvfp4_qdq(ptr(QDQ_INPUT), 32, 64.0, ptr(packed), ptr(scales), ptr(dq)) == 0
    assert np.array_equal(packed, QDQ_PACKED) and np.array_equal(scales, QDQ_SCALES)
    assert np.array_equal(bits(dq), QDQ_DEQUANT_BITS)


def test_matvec_golden_bits(oracle):
    # tests/test_nvfp4.c:92-105: weights 0x22 / 0xa2, scales 0x38, divisor 1, g = 64
    w = np.concatenate([np.full(16, 0x22, np.uint8), np.full(16, 0xa2, np.uint8)])
    ws = np.full(4, 0x38, np.uint8)
    out = np.zeros(2, np.float32)
    xp = np.zeros(16, np.uint8); xs = np.zeros(2, np.uint8); xd = np.zeros(32, np.float32)
    assert oracle.orc_nvfp4_matvec(ptr(w), ptr(ws), 1.0, 64.0, 2, 32, ptr(QDQ_INPUT), ptr(out),
                                   ptr(xp), ptr(xs), ptr(xd)) == 0
    assert list(bits(out)) == [0xc0d00000, 0xc0f00000]


def test_qdq_rejects(oracle):
    p = np.zeros(16, np.uint8); s = np.zeros(2, np.uint8); d = np.zeros(32, np.float32)
    x = QDQ_INPUT.copy()
    assert oracle.orc_nvfp4_qdq(ptr(x), 24, 64.0, ptr(p), ptr(s), ptr(d)) == -1
    assert oracle.orc_nvfp4_qdq(ptr(x), 32, 0.0, ptr(p), ptr(s), ptr(d)) == -1
    assert oracle.orc_nvfp4_qdq(ptr(x), 32, float("inf"), ptr(p), ptr(s), ptr(d)) == -1
    x[3] = np.inf
    assert oracle.orc_nvfp4_qdq(ptr(x), 32, 64.0, ptr(p), ptr(s), ptr(d)) == -1
    z = np.zeros(32, np.float32)
    assert oracle.orc_nvfp4_qdq(ptr(z), 32, 64.0, ptr(p), ptr(s), ptr(d)) == 0
    assert not p.any() and not s.any() and not bits(d).any()


def test_row_against_dequantised_dot(oracle):
    R, Cc = 6, 256
    packed, scales = synth.nvfp4_tensor(R, Cc, 3)
    x = synth.activations(Cc, 1, 4)[0]
    w = np.zeros((R, Cc), np.float32)
    assert oracle.orc_nvfp4_dequant_weights(ptr(packed), ptr(scales), 2688.0, R, Cc, ptr(w)) == 0
    out = np.zeros(R, np.float32)
    assert oracle.orc_nvfp4_matvec_weights_only(ptr(packed), ptr(scales), 2688.0, R, Cc, ptr(x), ptr(out)) == 0
    f = np.float32
    acc = np.zeros((R, 32), f)
    for c in range(Cc):
        acc[:, c & 31] = (acc[:, c & 31] + (w[:, c] * x[c]).astype(f)).astype(f)
    part = np.zeros((R, 4), f)
    for a in range(8):
        part = (part + acc[:, 4 * a:4 * a + 4]).astype(f)
    want = ((part[:, 0] + part[:, 2]).astype(f) + (part[:, 1] + part[:, 3]).astype(f)).astype(f)
    assert np.array_equal(bits(out), bits(want))
    # decode table against torch's OCP tables
    torch = pytest.importorskip("torch")
    e4 = torch.from_numpy(scales.copy()).view(torch.float8_e4m3fn).float().numpy().reshape(R, Cc // 16)
    e2 = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, 0, -.5, -1, -1.5, -2, -3, -4, -6], f)
    codes = np.stack([packed & 15, packed >> 4], axis=1).reshape(R, Cc)
    wg = f(1.0) / f(2688.0)
    expect = (e2[codes] * np.repeat((e4 * wg).astype(f), 16, axis=1)).astype(f)
    assert np.array_equal(bits(w), bits(expect))


# ---- against the reference's own sources, when they have been compiled ----

def test_encode_equals_compiled_reference(oracle, reference):
    grid = [oracle.orc_e4m3fn(c) for c in range(0x7f)]
    a = C.c_uint8(0); b = C.c_uint8(0)
    for v in np.concatenate([_probe_points(grid), synth.rng(9).uniform(-500, 500, 5000).astype(np.float32)]):
        assert oracle.orc_e4m3fn_encode(float(v), C.byref(a)) == reference.salt_nvfp4_e4m3fn_encode(float(v), C.byref(b))
        assert a.value == b.value
    for code in range(256):
        x, y = oracle.orc_e4m3fn(code), reference.salt_nvfp4_e4m3fn(code)
        assert (np.isnan(x) and np.isnan(y)) or bits(np.float32(x)) == bits(np.float32(y))


@pytest.mark.parametrize("g", [64.0, 1.0, 37.5, 2688.0, 1e-3])
def test_qdq_equals_compiled_reference(oracle, reference, g):
    Cc = 4096
    x = synth.activations(Cc, 1, 17)[0]
    x[100:116] = 0; x[200] = 1e-30; x[300] = 3e4
    outs = []
    for fn in (oracle.orc_nvfp4_qdq, reference.salt_nvfp4_quantize_input_reference):
        p = np.zeros(Cc // 2, np.uint8); s = np.zeros(Cc // 16, np.uint8); d = np.zeros(Cc, np.float32)
        assert fn(ptr(x), Cc, g, ptr(p), ptr(s), ptr(d)) == 0
        outs.append((p, s, bits(d)))
    for a, b in zip(*outs):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("divisor", [1.0, 2688.0])
def test_matvec_equals_compiled_reference(oracle, reference, divisor):
    R, Cc = 48, 2816
    packed, scales = synth.nvfp4_tensor(R, Cc, 31)
    x = synth.activations(Cc, 1, 32)[0]
    res = []
    for fn in (oracle.orc_nvfp4_matvec, reference.salt_nvfp4_matvec_reference):
        out = np.zeros(R, np.float32)
        xp = np.zeros(Cc // 2, np.uint8); xs = np.zeros(Cc // 16, np.uint8); xd = np.zeros(Cc, np.float32)
        assert fn(ptr(packed), ptr(scales), divisor, 64.0, R, Cc, ptr(x), ptr(out), ptr(xp), ptr(xs), ptr(xd)) == 0
        res.append(bits(out))
    assert np.array_equal(res[0], res[1])
