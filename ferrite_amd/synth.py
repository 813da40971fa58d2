"""Seeded synthetic inputs for the MoE FFN layer.

The generator is counter based (splitmix64 over an index), so any slice of any tensor can be produced
independently and identically on every machine; it plays the role of the reference's seeded
xorshift64*/Box-Muller `random_weights` (crates/ferrite-model/src/weights.rs:198-255) for a layer whose
expert weights are MXFP4.

Distributions (seed 0 unless stated):
  activations      f32 ~ N(0,1), optionally rounded to bf16 (round-to-nearest-even)
  expert weights   e2m1 codes uniform over the 16 codes (raw uniform bytes, two codes per byte, low nibble
                   = even column), one e8m0 scale byte per 32 columns drawn from {119, 120} (2^-8, 2^-7):
                   dequantised std ~= 0.018
  router weight    f32 ~ N(0, 0.02);  correction bias f32 ~ N(0, 0.01), or a Zipf(s) ranking
"""
from __future__ import annotations

from dataclasses import dataclass, field, replace
from typing import Dict, Optional

import numpy as np

_U64 = np.uint64
_GOLD = _U64(0x9E3779B97F4A7C15)
_M1 = _U64(0xBF58476D1CE4E5B9)
_M2 = _U64(0x94D049BB133111EB)


def splitmix64(x: np.ndarray) -> np.ndarray:
    """The splitmix64 finaliser applied elementwise to a uint64 array (wrapping arithmetic)."""
    with np.errstate(over="ignore"):
        z = (x + _GOLD).astype(_U64)
        z = (z ^ (z >> _U64(30))) * _M1
        z = (z ^ (z >> _U64(27))) * _M2
        z = z ^ (z >> _U64(31))
    return z


def _stream(seed: int, stream: int, start: int, count: int) -> np.ndarray:
    """`count` uint64 values of stream `stream`, beginning at element `start`."""
    with np.errstate(over="ignore"):
        base = splitmix64(np.array([seed * 0x10001 + 0x51ED27], dtype=_U64))[0] ^ splitmix64(
            np.array([stream + 0x7F4A7C15], dtype=_U64)
        )[0]
        idx = np.arange(start, start + count, dtype=_U64)
        return splitmix64(idx * _GOLD + base)


def random_bytes(seed: int, stream: int, nbytes: int) -> np.ndarray:
    """Uniform bytes; byte b of the stream is byte (b % 8) of the little-endian word b // 8."""
    nwords = (nbytes + 7) // 8
    out = np.empty(nwords * 8, dtype=np.uint8)
    chunk = 1 << 24
    for s in range(0, nwords, chunk):
        c = min(chunk, nwords - s)
        out[s * 8:(s + c) * 8] = _stream(seed, stream, s, c).view(np.uint8)
    return out[:nbytes]


def random_normal(seed: int, stream: int, count: int, std: float = 1.0) -> np.ndarray:
    """f32 normals by Box-Muller on two 53-bit uniforms per value (computed in float64)."""
    out = np.empty(count, dtype=np.float32)
    chunk = 1 << 22
    for s in range(0, count, chunk):
        c = min(chunk, count - s)
        r = _stream(seed, stream, 2 * s, 2 * c)
        u1 = ((r[0::2] >> _U64(11)).astype(np.float64) + 1.0) / 9007199254740993.0  # (0, 1)
        u2 = (r[1::2] >> _U64(11)).astype(np.float64) / 9007199254740992.0
        out[s:s + c] = (np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2) * std).astype(np.float32)
    return out


def round_to_bf16(x: np.ndarray) -> np.ndarray:
    """Round f32 to the nearest bf16 (ties to even) and return it as f32."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    return (r & np.uint32(0xFFFF0000)).view(np.float32)


@dataclass(frozen=True)
class MoeConfig:
    """Shape of one MoE FFN layer (the fields of the reference's text config that the path reads:
    crates/ferrite-model/src/config.rs:24-86, plus the group fields the north-star configs add)."""

    n: int                 # tokens
    hidden: int            # H
    n_experts: int         # E routed experts
    topk: int              # k
    inter: int             # I = moe_intermediate
    shared_inter: int      # Is (the reference uses moe_intermediate for the shared expert)
    n_group: int = 1
    topk_group: int = 1
    routed_scaling: float = 2.5
    swiglu_limit: float = 10.0
    act_bf16: bool = False  # activations rounded to bf16
    bias_zipf: float = 0.0  # > 0: correction bias from a Zipf(s) ranking instead of N(0, 0.01)
    name: str = ""

    def with_tokens(self, n: int) -> "MoeConfig":
        return replace(self, n=n)


# The five workload shapes of the benchmark plan.
CONFIGS: Dict[str, MoeConfig] = {
    "c0": MoeConfig(8, 256, 16, 4, 128, 128, 4, 2, name="c0-tiny"),
    "c1": MoeConfig(32, 4096, 128, 8, 1536, 1536, 8, 4, act_bf16=True, name="c1-decode32"),
    "c2": MoeConfig(4096, 4096, 128, 8, 1536, 1536, 8, 4, act_bf16=True, name="c2-prefill4096"),
    "c3": MoeConfig(8192, 7168, 256, 8, 2048, 2048, 8, 4, act_bf16=True, bias_zipf=1.1, name="c3-dsv3-skew"),
    "c4": MoeConfig(192, 4096, 128, 8, 1536, 1536, 8, 4, act_bf16=True, name="c4-decode192x42"),
}

# stream ids
_S_X, _S_ROUTER, _S_BIAS = 1, 2, 3
_S_GATE, _S_UP, _S_DOWN, _S_SH = 10, 20, 30, 40
ZIPF_ALPHA = 0.055  # bias = ZIPF_ALPHA * (ln p_rank - mean ln p); see zipf_bias


def mxfp4_matrix(seed: int, stream: int, n_mat: int, rows: int, cols: int):
    """`n_mat` stacked MXFP4 matrices in checkpoint layout: codes [n_mat, rows, cols/2] u8 and
    e8m0 scales [n_mat, rows, cols/32] u8."""
    codes = random_bytes(seed, stream, n_mat * rows * (cols // 2)).reshape(n_mat, rows, cols // 2)
    sbits = random_bytes(seed, stream + 1, n_mat * rows * (cols // 32)).reshape(n_mat, rows, cols // 32)
    scales = (np.uint8(119) + (sbits & np.uint8(1))).astype(np.uint8)
    return codes, scales


def zipf_bias(seed: int, n_experts: int, s: float, alpha: float = ZIPF_ALPHA) -> np.ndarray:
    """Correction bias that skews expert popularity along a Zipf(s) ranking: experts are ranked by a
    seeded permutation, rank r gets target mass p_r ~ r^-s, bias = alpha * (ln p_r - mean ln p)."""
    order = np.argsort(_stream(seed, _S_BIAS, 0, n_experts), kind="stable")
    rank = np.empty(n_experts, dtype=np.int64)
    rank[order] = np.arange(1, n_experts + 1)
    lp = -s * np.log(rank.astype(np.float64))
    return (alpha * (lp - lp.mean())).astype(np.float32)


@dataclass
class MoeInputs:
    cfg: MoeConfig
    x: np.ndarray            # [n, H] f32
    router_w: np.ndarray     # [E, H] f32
    router_bias: np.ndarray  # [E] f32
    gate_w: np.ndarray       # [E, I, H/2] u8
    gate_s: np.ndarray       # [E, I, H/32] u8
    up_w: np.ndarray
    up_s: np.ndarray
    down_w: np.ndarray       # [E, H, I/2] u8
    down_s: np.ndarray       # [E, H, I/32] u8
    sh_gate_w: np.ndarray    # [1, Is, H/2]
    sh_gate_s: np.ndarray
    sh_up_w: np.ndarray
    sh_up_s: np.ndarray
    sh_down_w: np.ndarray    # [1, H, Is/2]
    sh_down_s: np.ndarray
    extra: dict = field(default_factory=dict)


def make_activations(cfg: MoeConfig, seed: int = 0, n: Optional[int] = None) -> np.ndarray:
    n = cfg.n if n is None else n
    x = random_normal(seed, _S_X, n * cfg.hidden).reshape(n, cfg.hidden)
    return round_to_bf16(x) if cfg.act_bf16 else x


def make_inputs(cfg: MoeConfig, seed: int = 0, layer: int = 0) -> MoeInputs:
    """All tensors of one layer.  `layer` offsets the weight streams so stacked layers differ."""
    E, H, I, Is = cfg.n_experts, cfg.hidden, cfg.inter, cfg.shared_inter
    o = layer * 1000
    x = make_activations(cfg, seed)
    router_w = random_normal(seed, _S_ROUTER + o, E * H, 0.02).reshape(E, H)
    if cfg.bias_zipf > 0:
        bias = zipf_bias(seed + layer, E, cfg.bias_zipf)
    else:
        bias = random_normal(seed, _S_BIAS + o, E, 0.01)
    gate_w, gate_s = mxfp4_matrix(seed, _S_GATE + o, E, I, H)
    up_w, up_s = mxfp4_matrix(seed, _S_UP + o, E, I, H)
    down_w, down_s = mxfp4_matrix(seed, _S_DOWN + o, E, H, I)
    sgw, sgs = mxfp4_matrix(seed, _S_SH + o, 1, Is, H)
    suw, sus = mxfp4_matrix(seed, _S_SH + 2 + o, 1, Is, H)
    sdw, sds = mxfp4_matrix(seed, _S_SH + 4 + o, 1, H, Is)
    return MoeInputs(cfg, x, router_w, bias, gate_w, gate_s, up_w, up_s, down_w, down_s,
                     sgw, sgs, suw, sus, sdw, sds)
