"""Affine-Q4 matvec on the MI355X through the C ABI, bit-for-bit against the
CPU checker and the committed reference fixtures."""
import numpy as np
import pytest

from golden import cases
from oracle_lib import bits, host_threads, ptr

pytestmark = pytest.mark.gpu
synth = cases.synth


@pytest.fixture(scope="module")
def gpu(pkg):
    pkg.lib.init()
    return pkg.lib


def oracle_batch(oracle, vals, scales, biases, R, C, xs):
    ys = np.zeros((xs.shape[0], R), np.float32)
    for t in range(xs.shape[0]):
        assert oracle.orc_q4_matvec_threads(ptr(vals), ptr(scales), ptr(biases), R, C, ptr(xs[t]), ptr(ys[t]),
                                            host_threads()) == 0
    return ys


def test_converters_decode_as_assumed(gpu):
    lib = gpu.load()
    fp8 = np.zeros(256, np.float32); fp4 = np.zeros(512, np.float32)
    assert lib.salt_mi355_converter_tables(ptr(fp8), ptr(fp4)) == 0
    unit = fp8[1]
    print("fp8 converter unit", unit, flush=True)
    assert unit in (2.0 ** -9, 2.0 ** -10)
    assert np.array_equal(fp8[:16], np.arange(16, dtype=np.float32) * unit)
    mag = np.array([0, .5, 1, 1.5, 2, 3, 4, 6], np.float32)
    codes = np.stack([np.arange(256) & 15, np.arange(256) >> 4], axis=1).ravel()
    want = np.where(codes & 8, -mag[codes & 7], mag[codes & 7])
    assert np.array_equal(fp4, want.astype(np.float32))


@pytest.mark.parametrize("chains", [8, 4, 2])
@pytest.mark.parametrize("R,C,B", [(64, 64, 1), (130, 256, 2), (704, 2816, 1), (2816, 704, 3), (65, 8192, 4),
                                   (1, 64, 1), (63, 1088, 1)])
def test_tiled_kernel_matches_checker(gpu, oracle, R, C, B, chains):
    print(f"case R={R} C={C} B={B} chains={chains}", flush=True)
    vals, scales, biases = synth.q4_tensor(R, C, R * 31 + C)
    xs = synth.activations(C, B, R + C + B)
    got = gpu.q4_matvec(vals, scales, biases, R, C, xs, chains)
    assert np.array_equal(bits(got), bits(oracle_batch(oracle, vals, scales, biases, R, C, xs)))


@pytest.mark.parametrize("case", cases.Q4_CASES, ids=lambda c: c[0])
def test_reference_fixtures(gpu, case):
    name, R, C, B, wseed, xseed, stride = case
    print("fixture", name, flush=True)
    fx = cases.load("q4_matvec.npz")
    vals, scales, biases, xs = cases.q4_case_inputs(R, C, B, wseed, xseed)
    assert cases.digest(vals, scales, biases, xs) == str(fx[name + ".digest"])
    got = gpu.q4_matvec(vals[:R * C // 8] if (R * C) % 8 == 0 else vals, scales, biases, R, C, xs)
    assert np.array_equal(bits(got)[:, fx[name + ".rows"]], fx[name + ".y_bits"])


@pytest.mark.parametrize("offset", [4, 8, 12, 24])
def test_tiled_kernel_with_dword_aligned_values(gpu, oracle, offset):
    """Packed values that start 4, 8 or 12 bytes past a multiple of 16 (the engine's expert pool file puts every tensor
    24 bytes past a page boundary): same bits, still the tiled kernel."""
    print("q4 value offset", offset, flush=True)
    for R, C, B in [(2816, 704, 1), (130, 2816, 2)]:
        vals, scales, biases = synth.q4_tensor(R, C, offset + R)
        xs = synth.activations(C, B, 9)
        got = gpu.q4_matvec(vals, scales, biases, R, C, xs, value_offset=offset)
        assert np.array_equal(bits(got), bits(oracle_batch(oracle, vals, scales, biases, R, C, xs)))


def test_generic_kernel_odd_columns_and_null_bias(gpu, oracle):
    for R, C, B in [(8, 200, 1), (9, 96, 2), (70, 40, 1)]:
        print(f"generic R={R} C={C} B={B}", flush=True)
        pad = (-(R * C)) % 64
        vals, scales, biases = synth.q4_tensor(1, R * C + pad, R + C)
        xs = synth.activations(C, B, 3)
        got = gpu.q4_matvec(vals, scales, biases, R, C, xs)
        assert np.array_equal(bits(got), bits(oracle_batch(oracle, vals, scales, biases, R, C, xs)))
    vals, scales, _ = synth.q4_tensor(64, 128, 5)
    xs = synth.activations(128, 1, 6)
    got = gpu.q4_matvec(vals, scales, None, 64, 128, xs)
    assert np.array_equal(bits(got), bits(oracle_batch(oracle, vals, scales, None, 64, 128, xs)))


def test_extreme_scales_subnormals_and_zero(gpu, oracle):
    R, C = 64, 256
    vals, scales, biases = synth.q4_tensor(R, C, 77)
    scales = scales.copy(); biases = biases.copy()
    scales[0] = 0x7F00          # 1.7e38: scale * 2^9 would overflow
    biases[0] = 0xFF00          # -1.7e38
    scales[1] = 0x0001          # bf16 subnormal
    scales[2] = 0x0080          # smallest normal
    biases[2] = 0x8003          # negative subnormal
    scales[5] = 0x7E80          # 8.5e37, large but scale*2^9 still overflows
    xs = synth.activations(C, 2, 78)
    xs[1] *= np.float32(1e-30)
    for chains in (8, 4, 2):
        got = gpu.q4_matvec(vals, scales, biases, R, C, xs, chains)
        want = oracle_batch(oracle, vals, scales, biases, R, C, xs)
        same = (bits(got) == bits(want)) | (np.isnan(got) & np.isnan(want))
        assert same.all(), chains
    zero = gpu.q4_matvec(vals, synth.q4_tensor(R, C, 77)[1], biases, R, C, np.zeros((1, C), np.float32))
    assert not bits(zero).any()


def test_many_jobs_one_launch(gpu, oracle, pkg):
    import ctypes as C_
    lib = gpu.load()
    Ccols, tokens = 512, 2
    rows = [64, 200, 1, 129, 704]
    hold, jobs, want = [], (pkg.lib.Q4Job * len(rows))(), []
    for j, R in enumerate(rows):
        vals, scales, biases = synth.q4_tensor(R, Ccols, 900 + j)
        xs = synth.activations(Ccols, tokens, 950 + j)
        bufs = [pkg.lib.DeviceBuffer.from_host(a) for a in (vals, scales, biases, xs)]
        out = pkg.lib.DeviceBuffer(tokens * R * 4, fill=0xFF)
        hold.append((bufs, out))
        jobs[j] = pkg.lib.Q4Job(bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, bufs[3].ptr, out.ptr, R)
        want.append(oracle_batch(oracle, vals, scales, biases, R, Ccols, xs))
    stream = lib.salt_mi355_stream()
    for chains in (0, 8, 2):
        assert lib.salt_mi355_q4_jobs_dev(jobs, len(rows), Ccols, tokens, chains, stream) == 0
        assert lib.salt_mi355_stream_sync(stream) == 0
        for j, R in enumerate(rows):
            got = hold[j][1].to_host(np.float32).reshape(tokens, R)
            assert np.array_equal(bits(got), bits(want[j])), (chains, j)


def test_rejects_bad_arguments(gpu):
    lib = gpu.load()
    assert lib.salt_mi355_q4_matvec_dev(None, None, None, 4, 64, 1, None, None, 0, None) == -1
    buf = gpu.DeviceBuffer(4096)
    assert lib.salt_mi355_q4_matvec_dev(buf.ptr, buf.ptr, None, 0, 64, 1, buf.ptr, buf.ptr, 0, None) == -1
    assert lib.salt_mi355_q4_matvec_dev(buf.ptr, buf.ptr, None, 4, 64, 0, buf.ptr, buf.ptr, 0, None) == -1
    assert lib.salt_mi355_q4_matvec_dev(buf.ptr, buf.ptr, None, 4, 64, 1, buf.ptr, buf.ptr, 3, None) == -1
    assert b"chains" in lib.salt_mi355_last_error()
