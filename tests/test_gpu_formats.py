"""The formats themselves on the device: affine-Q4 decode, NVFP4 weight dequantisation and the fixture router, each
bit for bit against the CPU checker (pinned by the reference's own known answers and by fixtures written from the
compiled reference: tests/test_oracle_q4.py, tests/test_oracle_nvfp4.py, tests/golden/router.npz)."""
import numpy as np
import pytest

from golden import cases
from oracle_lib import bits, ptr

pytestmark = pytest.mark.gpu
synth = cases.synth


def test_q4_decode_matches_the_checker_and_the_reference_known_answers(pkg, oracle):
    gpu = pkg.lib
    lib = gpu.init()
    stream = lib.salt_mi355_stream()
    # reference tests/test_kernels.c:357-392: codes k % 16 with scale 1 decode to their own value; element 64 takes the
    # second group's scale: 5 * 2.0
    n = 128
    q = (np.arange(n) % 16).astype(np.uint8)
    q[64] = 5
    vals = synth.pack_nibbles_u32(q)
    scales = synth.f32_to_bf16_bits(np.array([1.0, 2.0], np.float32))
    biases = synth.f32_to_bf16_bits(np.array([0.0, 0.0], np.float32))
    for use_bias in (True, False):
        dv, ds, db = (gpu.DeviceBuffer.from_host(a) for a in (vals, scales, biases))
        out = gpu.DeviceBuffer(n * 4, fill=0xFF)
        gpu.check(lib.salt_mi355_q4_decode_dev(dv.ptr, ds.ptr, db.ptr if use_bias else None, n, out.ptr, stream), "decode")
        gpu.check(lib.salt_mi355_stream_sync(stream), "sync")
        got = out.to_host(np.float32)
        assert got[17] == 1.0 and got[63] == 15.0 and got[64] == 10.0 and got[65] == 2.0
    # seeded tensor, byte-misaligned pointers
    R, Cc = 37, 192
    vals, scales, biases = synth.q4_tensor(R, Cc, 3)
    n = R * Cc
    want = np.zeros(n, np.float32)
    oracle.orc_q4_decode(ptr(vals), ptr(scales), ptr(biases), n, ptr(want))
    for offset in (0, 1, 3):
        dv = gpu.DeviceBuffer(vals.nbytes + 8, fill=0); dv.upload(vals, offset)
        ds = gpu.DeviceBuffer(scales.nbytes + 8, fill=0); ds.upload(scales, offset)
        db = gpu.DeviceBuffer(biases.nbytes + 8, fill=0); db.upload(biases, offset)
        out = gpu.DeviceBuffer(n * 4, fill=0xFF)
        gpu.check(lib.salt_mi355_q4_decode_dev(dv.at(offset), ds.at(offset), db.at(offset), n, out.ptr, stream), "decode")
        gpu.check(lib.salt_mi355_stream_sync(stream), "sync")
        assert np.array_equal(bits(out.to_host(np.float32)), bits(want))
    assert lib.salt_mi355_q4_decode_dev(None, ds.ptr, None, 8, out.ptr, stream) == -1


def test_nvfp4_weight_dequantisation_matches_the_checker(pkg, oracle):
    gpu = pkg.lib
    lib = gpu.init()
    stream = lib.salt_mi355_stream()
    R, Cc = 33, 160
    packed, scales = synth.nvfp4_tensor(R, Cc, 7)
    scales = scales.copy()
    scales[5] = 0x7F                                  # NaN scale code
    scales[6] = 0x00
    packed = packed.copy()
    packed[:8] = [0x80, 0x08, 0x88, 0xF7, 0x7F, 0x19, 0x91, 0x00]     # both signs of zero, the extremes
    for divisor in (1.0, 2688.0, -3.0):
        want = np.zeros(R * Cc, np.float32)
        assert oracle.orc_nvfp4_dequant_weights(ptr(packed), ptr(scales), divisor, R, Cc, ptr(want)) == 0
        dp, ds = gpu.DeviceBuffer.from_host(packed), gpu.DeviceBuffer.from_host(scales)
        out = gpu.DeviceBuffer(R * Cc * 4, fill=0xFF)
        gpu.check(lib.salt_mi355_nvfp4_dequant_weights_dev(dp.ptr, ds.ptr, divisor, R, Cc, out.ptr, stream), "dequant")
        gpu.check(lib.salt_mi355_stream_sync(stream), "sync")
        got = out.to_host(np.float32)
        finite = ~np.isnan(want)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(bits(got)[finite], bits(want)[finite])
    assert lib.salt_mi355_nvfp4_dequant_weights_dev(dp.ptr, ds.ptr, 0.0, R, Cc, out.ptr, stream) == -1
    assert lib.salt_mi355_nvfp4_dequant_weights_dev(dp.ptr, ds.ptr, 1.0, R, 24, out.ptr, stream) == -1


def test_fixture_router_matches_the_reference_fixtures_and_the_checker(pkg, oracle):
    gpu = pkg.lib
    lib = gpu.init()
    stream = lib.salt_mi355_stream()
    fx = cases.load("router.npz")

    def run(E, K, state, layer, locality):
        idx, w = gpu.DeviceBuffer(K * 4, fill=0xEE), gpu.DeviceBuffer(K * 4, fill=0xEE)
        gpu.check(lib.salt_mi355_router_fixture_dev(E, K, int(state), int(layer), float(locality), idx.ptr, w.ptr, stream),
                  "fixture router")
        gpu.check(lib.salt_mi355_stream_sync(stream), "sync")
        return idx.to_host(np.int32), w.to_host(np.float32)

    for i in range(len(fx["fx_states"])):                        # written from the compiled reference's salt_router
        idx, w = run(128, 8, fx["fx_states"][i], fx["fx_layers"][i], fx["fx_locality"][i])
        assert np.array_equal(idx, fx["fx_idx"][i]) and np.array_equal(bits(w), fx["fx_w_bits"][i])
    rng = synth.rng(5)
    for E, K in ((1, 1), (7, 7), (64, 3), (300, 17), (1024, 64)):
        for locality in (0.0, 0.75, 3.5):
            state, layer = int(rng.integers(0, 2 ** 63)), int(rng.integers(0, 60))
            want_idx, want_w = np.zeros(K, np.int32), np.zeros(K, np.float32)
            assert oracle.orc_router_fixture(ptr(want_idx), ptr(want_w), E, K, state, layer, locality) == 0
            idx, w = run(E, K, state, layer, locality)
            assert np.array_equal(idx, want_idx) and np.array_equal(bits(w), bits(want_w)), (E, K, locality)
    buf = gpu.DeviceBuffer(64)
    assert lib.salt_mi355_router_fixture_dev(8, 9, 1, 0, 0.0, buf.ptr, buf.ptr, stream) == -1
    assert lib.salt_mi355_router_fixture_dev(2000, 4, 1, 0, 0.0, buf.ptr, buf.ptr, stream) == -1
