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


def qdq_e4m3(a, block=32, pow2_scale=True):
    """Quantise-dequantise through e4m3 per `block` values with the reference's scale rule, as an independent
    statement: torch's float8_e4m3fn cast does the rounding (round to nearest even, 3 mantissa bits, subnormal step
    2^-9), the scale is 2^ceil(log2(amax / 448)) from an f32 division (crates/ferrite-models/src/dsv41/quant.rs:
    190-198) or amax / 448 itself (pow2_scale=False).  One reference quirk is applied by hand: a scaled magnitude in
    [7.5, 8) * 2^-9 encodes as the largest subnormal 7 * 2^-9, where round-to-nearest gives 2^-6 (quant.rs:108-112).
    Input is rounded to f32 first (the quantiser's input type); returns float64."""
    import torch
    a32 = np.asarray(a, np.float32)
    blk = a32.reshape(-1, block)
    amax = np.abs(blk).max(axis=1)
    if pow2_scale:
        q = amax / np.float32(448.0)                       # f32 division, as the reference computes it
        m, ex = np.frexp(q.astype(np.float64))             # q = m * 2^ex, m in [0.5, 1)
        e = np.where(m > 0.5, ex, ex - 1)                  # ceil(log2 q), exactly
        e = np.where(amax > 0, np.maximum(e, -126), -126)  # floored at the smallest normal
        scale = 2.0 ** e.astype(np.float64)
    else:
        scale = np.maximum(amax.astype(np.float64) / 448.0, 2.0 ** -126)
    y = blk.astype(np.float64) / scale[:, None]
    dq = torch.from_numpy(y.astype(np.float32)).to(torch.float8_e4m3fn).to(torch.float64).numpy()
    quirk = (np.abs(y) >= 7.5 / 512) & (np.abs(y) < 8.0 / 512)
    dq = np.where(quirk, np.sign(y) * 7.0 / 512, dq)
    return (dq * scale[:, None]).reshape(a32.shape)


def qdq_e4m3_x2(a):
    """Two-term form: the quantiser applied to x and then to what it leaves over (an f32 subtraction)."""
    a32 = np.asarray(a, np.float32)
    d1 = qdq_e4m3(a32)
    r = a32 - d1.astype(np.float32)
    return d1 + qdq_e4m3(r)


def expert(x, wg, wu, wd, limit, quant_act=None):
    g = np.minimum(x @ wg.T, limit)
    u = np.clip(x @ wu.T, -limit, limit)
    act = g / (1.0 + np.exp(-g)) * u
    if quant_act is not None:
        act = quant_act(act)
    return act @ wd.T


def moe_layer(inp, ids=None, probs=None, quant_x=None, quant_act=None):
    """float64 layer output; routing recomputed unless ids/probs are given.  quant_x / quant_act: what the expert
    GEMMs see in place of x and of the SwiGLU output (routing always sees x itself), the two places where the
    reference's device chain quantises (dsv41_quant_fp8 in front of the first GEMM, dsv41_swiglu_limit_q after the
    activation: crates/ferrite-models/src/dsv41/kernels.rs:97-108,586-598)."""
    cfg = inp.cfg
    x = inp.x.astype(np.float64)
    if ids is None:
        logits = x @ inp.router_w.astype(np.float64).T
        probs, ids = route(logits, inp.router_bias.astype(np.float64), cfg.topk, cfg.routed_scaling,
                           cfg.n_group, cfg.topk_group)
    xe = x if quant_x is None else quant_x(x)
    out = np.zeros_like(x)
    for e in np.unique(ids):
        wg, wu, wd = dequant(inp.gate_w[e], inp.gate_s[e]), dequant(inp.up_w[e], inp.up_s[e]), dequant(inp.down_w[e], inp.down_s[e])
        t, j = np.nonzero(ids == e)
        out[t] += probs[t, j][:, None] * expert(xe[t], wg, wu, wd, cfg.swiglu_limit, quant_act)
    out += expert(xe, dequant(inp.sh_gate_w[0], inp.sh_gate_s[0]), dequant(inp.sh_up_w[0], inp.sh_up_s[0]),
                  dequant(inp.sh_down_w[0], inp.sh_down_s[0]), cfg.swiglu_limit, quant_act)
    return out, probs, ids


def max_abs_rel(a, b):
    """max |a-b| / max |b| : the layer-output tolerance metric used throughout the tests."""
    return float(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)).max() / np.abs(b).max())
