"""Case tables and seeded inputs shared by the fixture generator
(make_golden.py) and the tests that read the fixtures."""
from __future__ import annotations

import hashlib

import numpy as np

from __graft_entry__ import load_package

synth = load_package().synth


def digest(*arrays) -> str:
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()



def pool_digest(pool, *rest) -> str:
    """Digest of a strided sample of a (large) expert pool plus small arrays."""
    return digest(pool[:: max(1, pool.size // (1 << 22))], *rest)


Q4_CASES = [
    # name, R, C, B, weight seed, x seed, row stride kept in the fixture
    ("cfg0_4096x4096_b1", 4096, 4096, 1, 0, 1000, 1),
    ("cfg1_2816x2816_b1", 2816, 2816, 1, 1, 1001, 1),
    ("cfg1_16384x2816_b1", 16384, 2816, 1, 2, 1002, 4),
    ("cfg1_2816x8192_b1", 2816, 8192, 1, 3, 1003, 1),
    ("cfg1_2816x2816_b4", 2816, 2816, 4, 4, 1004, 2),
    ("cfg1_16384x2816_b4", 16384, 2816, 4, 5, 1005, 16),
    ("cfg1_2816x8192_b4", 2816, 8192, 4, 6, 1006, 4),
    ("expert_gate_704x2816_b1", 704, 2816, 1, 7, 1007, 1),
    ("expert_down_2816x704_b1", 2816, 704, 1, 8, 1008, 1),
    ("odd_rows_705x2816_b3", 705, 2816, 3, 9, 1009, 1),
    ("tiny_3x64_b1", 3, 64, 1, 10, 1010, 1),
    ("wide_5x8192_b2", 5, 8192, 2, 11, 1011, 1),
]


def q4_case_inputs(R, C, B, wseed, xseed):
    pad = (-(R * C)) % 64
    vals, scales, biases = synth.q4_tensor(1, R * C + pad, wseed)
    xs = synth.activations(C, B, xseed)
    return vals, scales, biases, xs



NVFP4_QDQ_CASES = [("g64", 64.0, 501), ("g2688", 2688.0, 502), ("g0p37", 0.37, 503)]


def nvfp4_qdq_input(tag, seed):
    x = synth.activations(8192, 1, seed)[0]
    if tag == "g2688":
        x[64:80] = 0.0; x[100] = 50.0; x[200] = 1e-20
    return x


NVFP4_MATVEC_CASES = [
    # name, R, C, weight seed, x seed, stored divisor, input global scale
    ("cfg4_8192x8192_b1", 8192, 8192, 40, 541, 2688.0, 64.0),
    ("small_96x2816_div1", 96, 2816, 41, 542, 1.0, 64.0),
]


MOE_CASES = [
    # name, E, topk, hidden, routed, pool seed, logits seed, x seed
    ("gemma_e16", 16, 8, 2816, 704, 11, 611, 612),
    ("gemma_e128", 128, 8, 2816, 704, 12, 613, 614),
    ("small_e8", 8, 3, 256, 128, 13, 615, 616),
]



def moe_case_inputs(E, H, F, pseed, lseed, xseed):
    pool = synth.expert_pool(E, H, F, pseed)
    logits = synth.router_logits(E, lseed)
    x = synth.activations(H, 1, xseed)[0]
    return pool, logits, np.ones(E, np.float32), x


GROUP_CASES = [
    # name, T, E, topk, hidden, routed, run_batch (0 = per-expert run), seeds
    ("t24_e16_k4_many", 24, 16, 4, 256, 128, 5, 21, 721),
    ("t24_e16_k4_single", 24, 16, 4, 256, 128, 0, 21, 721),
    ("t6_e8_k2_gemma", 6, 8, 2, 2816, 704, 3, 22, 722),
]



def group_case_inputs(T, E, K, H, F, pseed, sseed):
    pool = synth.expert_pool(E, H, F, pseed)
    sel, w = synth.zipf_selection(T, E, K, 1.1, sseed)
    xs = synth.activations(H, T, sseed + 1)
    return pool, sel, w, xs


def load(name):
    from pathlib import Path
    return np.load(Path(__file__).resolve().parent / name, allow_pickle=False)
