"""The CPU checker against the committed fixtures (tests/golden/*.npz), which
hold outputs of the reference's own C sources on seeded inputs
(tests/golden/make_golden.py).  Runs without a GPU and without the reference."""
import ctypes as C

import numpy as np
import pytest

from golden import cases
from oracle_lib import ExpertGeometry, bits, host_threads, ptr

synth = cases.synth


@pytest.mark.parametrize("case", cases.Q4_CASES, ids=lambda c: c[0])
def test_q4_matvec(oracle, case):
    name, R, Cc, B, wseed, xseed, stride = case
    fx = cases.load("q4_matvec.npz")
    vals, scales, biases, xs = cases.q4_case_inputs(R, Cc, B, wseed, xseed)
    assert cases.digest(vals, scales, biases, xs) == str(fx[name + ".digest"])
    ys = np.zeros((B, R), np.float32)
    for t in range(B):
        assert oracle.orc_q4_matvec_threads(ptr(vals), ptr(scales), ptr(biases), R, Cc, ptr(xs[t]), ptr(ys[t]),
                                            host_threads()) == 0
    assert np.array_equal(bits(ys)[:, fx[name + ".rows"]], fx[name + ".y_bits"])


def test_bitmath(oracle):
    fx = cases.load("bitmath.npz")
    x = fx["x_bits"].view(np.float32)
    for fn, key in ((oracle.orc_expf, "expf_bits"), (oracle.orc_tanhf, "tanhf_bits"),
                    (oracle.orc_gelu_tanh, "gelu_bits")):
        got = np.array([fn(float(v)) for v in x], np.float32)
        assert np.array_equal(bits(got), fx[key]), key


def test_router_topk_and_fixture_router(oracle):
    fx = cases.load("router.npz")
    logits = fx["logits_bits"].view(np.float32); scale = fx["scale_bits"].view(np.float32)
    N, E = logits.shape
    K = fx["selected"].shape[1]
    for i in range(N):
        sel = np.zeros(K, np.int32); w = np.zeros(K, np.float32)
        assert oracle.orc_router_topk(ptr(np.ascontiguousarray(logits[i])), ptr(np.ascontiguousarray(scale[i])),
                                      E, K, ptr(sel), ptr(w)) == 0
        assert np.array_equal(sel, fx["selected"][i]) and np.array_equal(bits(w), fx["weight_bits"][i])
    for i in range(len(fx["fx_states"])):
        idx = np.zeros(8, np.int32); w = np.zeros(8, np.float32)
        assert oracle.orc_router_fixture(ptr(idx), ptr(w), 128, 8, int(fx["fx_states"][i]), int(fx["fx_layers"][i]),
                                         float(fx["fx_locality"][i])) == 0
        assert np.array_equal(idx, fx["fx_idx"][i]) and np.array_equal(bits(w), fx["fx_w_bits"][i])


def test_nvfp4_encode_and_qdq(oracle):
    fx = cases.load("nvfp4.npz")
    code = C.c_uint8(0)
    for v, want in zip(fx["enc_x_bits"].view(np.float32), fx["enc_codes"]):
        assert oracle.orc_e4m3fn_encode(float(v), C.byref(code)) == 0 and code.value == want
        assert oracle.orc_e4m3fn_encode_rne(float(v)) == want
    for tag, g, seed in cases.NVFP4_QDQ_CASES:
        x = cases.nvfp4_qdq_input(tag, seed)
        assert cases.digest(x) == str(fx[f"qdq_{tag}.digest"])
        p = np.zeros(4096, np.uint8); s = np.zeros(512, np.uint8); d = np.zeros(8192, np.float32)
        assert oracle.orc_nvfp4_qdq(ptr(x), 8192, g, ptr(p), ptr(s), ptr(d)) == 0
        assert np.array_equal(p, fx[f"qdq_{tag}.packed"]) and np.array_equal(s, fx[f"qdq_{tag}.scales"])
        assert np.array_equal(bits(d), fx[f"qdq_{tag}.dequant_bits"])


@pytest.mark.parametrize("case", cases.NVFP4_MATVEC_CASES, ids=lambda c: c[0])
def test_nvfp4_matvec(oracle, case):
    name, R, Cc, wseed, xseed, divisor, g = case
    fx = cases.load("nvfp4.npz")
    packed, scales = synth.nvfp4_tensor(R, Cc, wseed)
    x = synth.activations(Cc, 1, xseed)[0]
    assert cases.digest(packed, scales, x) == str(fx[name + ".digest"])
    rows = R if R <= 512 else 512          # the scalar row costs ~15 us per 1k columns
    y = np.zeros(rows, np.float32)
    xp = np.zeros(Cc // 2, np.uint8); xs = np.zeros(Cc // 16, np.uint8); xd = np.zeros(Cc, np.float32)
    assert oracle.orc_nvfp4_matvec(ptr(packed), ptr(scales), divisor, g, rows, Cc, ptr(x), ptr(y),
                                   ptr(xp), ptr(xs), ptr(xd)) == 0
    assert np.array_equal(bits(y), fx[name + ".y_bits"][:rows])


@pytest.mark.parametrize("case", [c for c in cases.MOE_CASES if c[1] <= 16], ids=lambda c: c[0])
def test_moe_decode_step(oracle, case):
    name, E, K, H, F, pseed, lseed, xseed = case
    fx = cases.load("moe_decode.npz")
    pool, logits, scale, x = cases.moe_case_inputs(E, H, F, pseed, lseed, xseed)
    assert cases.pool_digest(pool, logits, x) == str(fx[name + ".digest"])
    g = ExpertGeometry(H, F)
    sel = np.zeros(K, np.int32); w = np.zeros(K, np.float32)
    eo = np.zeros((K, H), np.float32); y = np.zeros(H, np.float32)
    assert oracle.orc_moe_decode_step(C.byref(g), ptr(pool), E, K, ptr(logits), ptr(scale), ptr(x), ptr(sel), ptr(w),
                                      ptr(eo), ptr(y), host_threads()) == 0
    assert np.array_equal(sel, fx[name + ".selected"]) and np.array_equal(bits(w), fx[name + ".weight_bits"])
    assert np.array_equal(bits(eo), fx[name + ".expert_out_bits"]) and np.array_equal(bits(y), fx[name + ".y_bits"])


@pytest.mark.parametrize("case", cases.GROUP_CASES, ids=lambda c: c[0])
def test_moe_group(oracle, case):
    name, T, E, K, H, F, run_batch, pseed, sseed = case
    fx = cases.load("moe_group.npz")
    pool, sel, w, xs = cases.group_case_inputs(T, E, K, H, F, pseed, sseed)
    assert cases.pool_digest(pool, xs) == str(fx[name + ".digest"])
    assert np.array_equal(sel, fx[name + ".selected"]) and np.array_equal(bits(w), fx[name + ".weight_bits"])
    g = ExpertGeometry(H, F)
    ys = np.zeros((T, H), np.float32); rows = np.zeros(E, np.int32)
    assert oracle.orc_moe_group(C.byref(g), ptr(pool), E, K, T, ptr(sel), ptr(w), ptr(xs), ptr(ys), ptr(rows),
                                host_threads()) == 0
    assert np.array_equal(bits(ys), fx[name + ".y_bits"])
    # the engine ran the used experts in ascending order with these row counts
    used = np.nonzero(rows)[0]
    assert np.array_equal(used, fx[name + ".run_experts"]) and np.array_equal(rows[used], fx[name + ".run_rows"])
