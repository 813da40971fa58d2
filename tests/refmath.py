"""Independent float64 NumPy statement of the layer (used to pin the oracle; not the oracle itself)."""
import numpy as np

FP4 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, 0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0])


def dequant(w, s):
    """codes [..., rows, cols/2] u8, scales [..., rows, cols/32] u8 -> float64 [..., rows, cols]"""
    codes = np.stack([w & 0xF, w >> 4], -1).reshape(*w.shape[:-1], w.shape[-1] * 2)
    return FP4[codes] * np.repeat(2.0 ** (s.astype(np.float64) - 127.0), 32, axis=-1)


def encode_exact(mat, scale_byte):
    """Encode a matrix whose entries are all FP4-representable multiples of 2^(scale_byte-127)."""
    q = mat / 2.0 ** (scale_byte - 127)
    codes = np.zeros(mat.shape, np.uint8)
    for c, v in enumerate(FP4):
        if c == 8:
            continue
        codes[q == v] = c
    assert np.array_equal(FP4[codes], q), "not representable"
    packed = (codes[..., 0::2] | (codes[..., 1::2] << 4)).astype(np.uint8)
    scales = np.full(mat.shape[:-1] + (mat.shape[-1] // 32,), scale_byte, np.uint8)
    return packed, scales


def route(logits, bias, topk, scaling, n_group=1, topk_group=1):
    n, e = logits.shape
    sig = 1.0 / (1.0 + np.exp(-logits))
    choice = sig + bias
    ids = np.zeros((n, topk), np.int64)
    probs = np.zeros((n, topk))
    for t in range(n):
        cand = list(range(e))
        if n_group > 1:
            gs = e // n_group
            gsc = [np.sort(choice[t, g * gs:(g + 1) * gs])[::-1][:2].sum() for g in range(n_group)]
            kept = sorted(range(n_group), key=lambda g: (-gsc[g], g))[:topk_group]
            cand = [j for j in cand if j // gs in kept]
        sel = sorted(cand, key=lambda j: (-choice[t, j], j))[:topk]
        ids[t] = sel
        probs[t] = sig[t, sel] / sig[t, sel].sum() * scaling
    return probs, ids


def expert(x, wg, wu, wd, limit):
    g = np.minimum(x @ wg.T, limit)
    u = np.clip(x @ wu.T, -limit, limit)
    return (g / (1.0 + np.exp(-g)) * u) @ wd.T


def moe_layer(inp, ids=None, probs=None):
    """float64 layer output; routing recomputed unless ids/probs are given."""
    cfg = inp.cfg
    x = inp.x.astype(np.float64)
    if ids is None:
        logits = x @ inp.router_w.astype(np.float64).T
        probs, ids = route(logits, inp.router_bias.astype(np.float64), cfg.topk, cfg.routed_scaling,
                           cfg.n_group, cfg.topk_group)
    out = np.zeros_like(x)
    for e in np.unique(ids):
        wg, wu, wd = dequant(inp.gate_w[e], inp.gate_s[e]), dequant(inp.up_w[e], inp.up_s[e]), dequant(inp.down_w[e], inp.down_s[e])
        t, j = np.nonzero(ids == e)
        out[t] += probs[t, j][:, None] * expert(x[t], wg, wu, wd, cfg.swiglu_limit)
    out += expert(x, dequant(inp.sh_gate_w[0], inp.sh_gate_s[0]), dequant(inp.sh_up_w[0], inp.sh_up_s[0]),
                  dequant(inp.sh_down_w[0], inp.sh_down_s[0]), cfg.swiglu_limit)
    return out, probs, ids


def max_abs_rel(a, b):
    """max |a-b| / max |b| : the layer-output tolerance metric used throughout the tests."""
    return float(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)).max() / np.abs(b).max())
