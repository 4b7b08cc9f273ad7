"""Float64 magnitudes behind the stated tolerances of the tolerance-class MoE tests: for one output, the sum of the
magnitudes of the terms that make it up.  Shared by the decode-step and the grouped-prefill tests."""
import numpy as np

from golden import cases

synth = cases.synth


def dequantised(pool, e, p, H, F):
    """Expert e's projection p (0 gate, 1 up, 2 down) as float64 [rows][cols]."""
    proj, n = synth.expert_proj_bytes(H, F), H * F
    at = (e * 3 + p) * proj
    vals = pool[at:at + n // 2].view(np.uint32)
    sc = synth.bf16_bits_to_f32(pool[at + n // 2:at + n // 2 + n // 32].view(np.uint16)).astype(np.float64)
    bi = synth.bf16_bits_to_f32(pool[at + n // 2 + n // 32:at + proj].view(np.uint16)).astype(np.float64)
    q = ((vals[:, None] >> (4 * np.arange(8, dtype=np.uint32))) & 15).reshape(-1).astype(np.float64)
    w = q * np.repeat(sc, 64) + np.repeat(bi, 64)
    return w.reshape((F, H) if p < 2 else (H, F))


def expert_activation(pool, e, xs, H, F):
    """h = gelu_tanh(gate) * up of expert e for the rows of xs, float64 [rows][F]."""
    gate, up = dequantised(pool, int(e), 0, H, F), dequantised(pool, int(e), 1, H, F)
    g = xs.astype(np.float64) @ gate.T
    return 0.5 * g * (1.0 + np.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3))) * (xs.astype(np.float64) @ up.T)


def down_term_magnitudes(pool, e, h, H, F):
    """sum_f |Wd[d][f] * h[f]| of expert e for every row of h, float64 [rows][H]."""
    return np.abs(h) @ np.abs(dequantised(pool, int(e), 2, H, F)).T


def group_term_magnitudes(pool, sel, w, xs, H, F):
    """M[token][d] = sum over the token's experts k of |w_k| * sum_f |Wd_k[d][f] * h_k[f]|."""
    T, K = sel.shape
    M = np.zeros((T, H))
    for e in np.unique(sel):
        tok, rank = np.nonzero(sel == e)
        h = expert_activation(pool, e, xs[tok], H, F)
        M[tok] += np.abs(w[tok, rank].astype(np.float64))[:, None] * down_term_magnitudes(pool, e, h, H, F)
    return M
