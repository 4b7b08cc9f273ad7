"""Seeded synthetic tensors shaped like the quantized decode workloads.

Everything here is plain numpy on the host: packed affine-Q4 matrices
(reference layout include/salt/kernels.h:117-130), routed-expert pools in the
Gemma slot layout (reference gemma4_text.c:73-79), NVFP4 matrices
(reference include/salt/nvfp4.h:37-46) and activations.  The same bytes feed
the CPU checker and the GPU library, so a seed names a test case.
"""
from __future__ import annotations

import numpy as np

GROUP = 64


def rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(int(seed)))


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even truncation of float32 to its top 16 bits."""
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    bits = bits + 0x7FFF + ((bits >> 16) & 1)
    return (bits >> 16).astype(np.uint16)


def bf16_bits_to_f32(h: np.ndarray) -> np.ndarray:
    return (h.astype(np.uint32) << 16).view(np.float32)


def pack_nibbles_u32(q: np.ndarray) -> np.ndarray:
    """q: flat uint8 array of 4-bit codes, length % 8 == 0 -> uint32 words,
    element k in bits [4*(k%8), 4*(k%8)+4) of word k//8."""
    q = q.reshape(-1, 8).astype(np.uint32)
    shifts = (4 * np.arange(8, dtype=np.uint32))[None, :]
    return np.bitwise_or.reduce(q << shifts, axis=1).astype(np.uint32)


def q4_tensor(R: int, C: int, seed: int):
    """Affine-Q4 matrix: q ~ U{0..15}; scale ~ U[0.005, 0.02] rounded to bf16;
    bias = -8*scale + N(0, 1e-3) rounded to bf16.  Returns (vals u32[R*C/8],
    scales u16[R*C/64], biases u16[R*C/64])."""
    assert (R * C) % GROUP == 0
    g = rng(seed)
    q = g.integers(0, 16, size=R * C, dtype=np.uint8)
    vals = pack_nibbles_u32(q)
    ngroups = R * C // GROUP
    scales = f32_to_bf16_bits(g.uniform(0.005, 0.02, size=ngroups).astype(np.float32))
    centre = np.float32(-8.0) * bf16_bits_to_f32(scales)
    jitter = g.normal(0.0, 1e-3, size=ngroups).astype(np.float32)
    biases = f32_to_bf16_bits(centre + jitter)
    return vals, scales, biases


def activations(C: int, B: int, seed: int) -> np.ndarray:
    """x ~ N(0,1), float32, shape [B, C]."""
    return rng(seed).standard_normal(size=(B, C)).astype(np.float32)


def expert_proj_bytes(hidden: int, routed: int) -> int:
    n = hidden * routed
    return n // 2 + 2 * (n // GROUP) * 2


def expert_slot_bytes(hidden: int, routed: int) -> int:
    return 3 * expert_proj_bytes(hidden, routed)


def expert_pool(n_experts: int, hidden: int, routed: int, seed: int) -> np.ndarray:
    """uint8 array of n_experts slots, each [gate|up|down], each projection
    [vals|scales|biases]; gate/up are routed x hidden, down is hidden x routed."""
    proj = expert_proj_bytes(hidden, routed)
    pool = np.empty(n_experts * 3 * proj, dtype=np.uint8)
    n = hidden * routed
    for e in range(n_experts):
        for p in range(3):
            vals, scales, biases = q4_tensor(routed if p < 2 else hidden,
                                             hidden if p < 2 else routed,
                                             seed * 1000003 + e * 3 + p)
            at = (e * 3 + p) * proj
            pool[at:at + n // 2] = vals.view(np.uint8)
            at += n // 2
            pool[at:at + scales.nbytes] = scales.view(np.uint8)
            at += scales.nbytes
            pool[at:at + biases.nbytes] = biases.view(np.uint8)
    return pool


def expert_views(pool: np.ndarray, expert: int, proj_index: int, hidden: int, routed: int):
    """(vals u32, scales u16, biases u16) views of one projection in a pool."""
    proj = expert_proj_bytes(hidden, routed)
    n = hidden * routed
    at = (expert * 3 + proj_index) * proj
    vals = pool[at:at + n // 2].view(np.uint32)
    meta = (n // GROUP) * 2
    scales = pool[at + n // 2:at + n // 2 + meta].view(np.uint16)
    biases = pool[at + n // 2 + meta:at + n // 2 + 2 * meta].view(np.uint16)
    return vals, scales, biases


def q8_tensor(R: int, C: int, seed: int):
    """(vals u8 [R*C], scales u16, biases u16): 8-bit affine, one bf16 scale and bias per 64 flat elements, values
    spread over about +-0.06."""
    g = rng(seed)
    vals = g.integers(0, 256, size=R * C, dtype=np.uint8)
    groups = (R * C + GROUP - 1) // GROUP
    scales = f32_to_bf16_bits(g.uniform(0.0003, 0.0006, groups).astype(np.float32))
    biases = f32_to_bf16_bits(g.uniform(-0.07, -0.04, groups).astype(np.float32))
    return vals, scales, biases


def ffn_layer(hidden: int, dense: int, routed: int, n_experts: int, topk: int, seed: int, pool=None) -> dict:
    """Weights of the feed-forward half of one decoder layer: norm weights, dense gate/up/down (affine Q4), the 8-bit
    router gate, router and per-expert scales, the expert pool (generated unless one is passed in)."""
    g = rng(seed)
    norm = lambda: (1.0 + 0.1 * g.standard_normal(hidden)).astype(np.float32)
    return {
        "hidden": hidden, "dense": dense, "routed": routed, "n_experts": n_experts, "topk": topk,
        "eps": np.float32(1e-6), "layer_scalar": np.float32(0.61),
        "pre_norm": norm(), "pre_norm_2": norm(), "post_norm_1": norm(), "post_norm_2": norm(), "post_norm": norm(),
        "router_scale": (1.0 + 0.3 * g.standard_normal(hidden)).astype(np.float32),
        "per_expert_scale": g.uniform(0.5, 2.0, n_experts).astype(np.float32),
        "dense_gate": q4_tensor(dense, hidden, seed * 7 + 1), "dense_up": q4_tensor(dense, hidden, seed * 7 + 2),
        "dense_down": q4_tensor(hidden, dense, seed * 7 + 3),
        "router": q8_tensor(n_experts, hidden, seed * 7 + 4),
        "pool": pool if pool is not None else expert_pool(n_experts, hidden, routed, seed * 7 + 5),
    }


def router_logits(n_experts: int, seed: int) -> np.ndarray:
    return rng(seed).standard_normal(size=n_experts).astype(np.float32)


def zipf_selection(batch: int, n_experts: int, topk: int, alpha: float, seed: int):
    """Per token `topk` distinct experts drawn without replacement with
    probability ~ 1/rank^alpha, sorted ascending; weights are the
    renormalised softmax of N(0,1) logits of the chosen experts."""
    g = rng(seed)
    p = 1.0 / np.arange(1, n_experts + 1, dtype=np.float64) ** alpha
    p /= p.sum()
    selected = np.empty((batch, topk), dtype=np.int32)
    for t in range(batch):
        selected[t] = np.sort(g.choice(n_experts, size=topk, replace=False, p=p))
    logits = g.standard_normal(size=(batch, topk))
    w = np.exp(logits - logits.max(axis=1, keepdims=True))
    w /= w.sum(axis=1, keepdims=True)
    return selected, w.astype(np.float32)


E4M3_SCALE_CODES = np.arange(0x08, 0x59, dtype=np.uint8)  # values 2^-6 .. 2^4


def nvfp4_tensor(R: int, C: int, seed: int):
    """NVFP4 matrix: E2M1 codes uniform over 16 codes packed two per byte (low
    nibble = even element); one E4M3FN scale per 16 columns, uniform over the
    codes whose value lies in [2^-6, 2^4].  Returns (packed u8[R*C/2],
    scales u8[R*C/16])."""
    assert C % 16 == 0
    g = rng(seed)
    codes = g.integers(0, 16, size=R * C, dtype=np.uint8).reshape(-1, 2)
    packed = (codes[:, 0] | (codes[:, 1] << 4)).astype(np.uint8)
    scales = E4M3_SCALE_CODES[g.integers(0, len(E4M3_SCALE_CODES), size=R * C // 16)]
    return packed, scales.astype(np.uint8)


def q4_bytes(R: int, C: int, B: int = 1) -> int:
    """Algorithmic bytes of one affine-Q4 matvec over B tokens."""
    return R * C // 2 + 2 * (R * C // GROUP) * 2 + 4 * B * (C + R)


def nvfp4_bytes(R: int, C: int, B: int = 1) -> int:
    return R * C // 2 + R * C // 16 + 4 + 4 * B * (C + R)


def moe_step_bytes(hidden: int, routed: int, n_experts: int, topk: int) -> int:
    return topk * expert_slot_bytes(hidden, routed) + 4 * hidden * 2 + 4 * n_experts
