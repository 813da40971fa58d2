"""ctypes binding of the CPU oracle (libferrite_oracle.so).  TEST INFRASTRUCTURE ONLY.

Imported by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg; never by the
ferrite_amd package.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libferrite_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (make -C oracle)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []), stdout=subprocess.DEVNULL)
    return _SO


class _Cfg(C.Structure):
    _fields_ = [("n", C.c_int), ("hidden", C.c_int), ("n_experts", C.c_int), ("topk", C.c_int),
                ("inter", C.c_int), ("shared_inter", C.c_int), ("n_group", C.c_int), ("topk_group", C.c_int),
                ("routed_scaling", C.c_float), ("swiglu_limit", C.c_float), ("act_mode", C.c_int),
                ("n_threads", C.c_int)]


class _Weights(C.Structure):
    _fields_ = [(k, C.c_void_p) for k in (
        "gate_w", "gate_s", "up_w", "up_s", "down_w", "down_s",
        "sh_gate_w", "sh_gate_s", "sh_up_w", "sh_up_s", "sh_down_w", "sh_down_s",
        "router_w", "router_bias")]


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_SO)
        L.fo_e2m1_decode.restype = C.c_float
        L.fo_e2m1_decode.argtypes = [C.c_uint8]
        L.fo_e2m1_encode.restype = C.c_uint8
        L.fo_e2m1_encode.argtypes = [C.c_float]
        L.fo_e4m3_decode.restype = C.c_float
        L.fo_e4m3_decode.argtypes = [C.c_uint8]
        L.fo_e4m3_encode.restype = C.c_uint8
        L.fo_e4m3_encode.argtypes = [C.c_float]
        L.fo_ue8m0_decode.restype = C.c_float
        L.fo_ue8m0_decode.argtypes = [C.c_uint8]
        L.fo_ue8m0_encode_pow2.restype = C.c_uint8
        L.fo_ue8m0_encode_pow2.argtypes = [C.c_int]
        L.fo_fast_log2_ceil.restype = C.c_int
        L.fo_fast_log2_ceil.argtypes = [C.c_float]
        L.fo_fast_pow2.restype = C.c_float
        L.fo_fast_pow2.argtypes = [C.c_int]
        L.fo_fast_round_scale.restype = C.c_float
        L.fo_fast_round_scale.argtypes = [C.c_float]
        vp = C.c_void_p
        L.fo_act_quant_fp8.restype = None
        L.fo_act_quant_fp8.argtypes = [vp, C.c_size_t, C.c_int, C.c_int, vp, vp]
        L.fo_act_quant_fp4.restype = None
        L.fo_act_quant_fp8_x2.argtypes = [vp, C.c_size_t, vp, vp, vp, vp]
        L.fo_act_quant_fp4.argtypes = [vp, C.c_size_t, C.c_int, C.c_int, vp, vp]
        L.fo_dequant_fp4_row32.restype = None
        L.fo_dequant_fp4_row32.argtypes = [vp, vp, C.c_size_t, C.c_size_t, vp]
        L.fo_matmul.argtypes = [vp, vp, vp, vp, C.c_int, C.c_int, C.c_int]
        L.fo_swiglu_limited.argtypes = [vp, C.c_float, vp, C.c_int, C.c_int]
        L.fo_rmsnorm.argtypes = [vp, vp, C.c_float, vp, C.c_int, C.c_int]
        L.fo_hc_post.argtypes = [vp, vp, vp, vp, vp, C.c_int, C.c_int, C.c_int]
        L.fo_moe_route.argtypes = [vp, vp, C.c_int, C.c_int, C.c_int, C.c_float, vp, vp]
        L.fo_moe_route_grouped.argtypes = [vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, vp, vp]
        L.fo_moe_route_grouped_nan.argtypes = [vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int,
                                               vp, vp]
        L.fo_expert_ffn.argtypes = [vp, vp, vp, vp, C.c_float, vp, C.c_int, C.c_int, C.c_int]
        L.fo_moe_permute.argtypes = [vp, C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, vp, vp]
        L.fo_moe_align_host.argtypes = [vp, C.c_int, C.c_int, C.c_int, C.c_int, vp, vp, vp]
        L.fo_moe_ffn_mxfp4.argtypes = [C.POINTER(_Cfg), C.POINTER(_Weights), vp, vp, C.c_int, vp, vp, vp, vp]
        _lib = L
    return _lib


def _p(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint8)


class OracleError(RuntimeError):
    pass


def _ck(rc: int, what: str):
    if rc != 0:
        raise OracleError(f"{what}: rc={rc}")


# ---- formats ----
def e2m1_decode(code: int) -> float: return lib().fo_e2m1_decode(code)
def e2m1_encode(x: float) -> int: return lib().fo_e2m1_encode(x)
def e4m3_decode(b: int) -> float: return lib().fo_e4m3_decode(b)
def e4m3_encode(x: float) -> int: return lib().fo_e4m3_encode(x)
def ue8m0_decode(b: int) -> float: return lib().fo_ue8m0_decode(b)
def ue8m0_encode_pow2(e: int) -> int: return lib().fo_ue8m0_encode_pow2(e)
def fast_log2_ceil(x: float) -> int: return lib().fo_fast_log2_ceil(x)
def fast_pow2(e: int) -> float: return lib().fo_fast_pow2(e)
def fast_round_scale(a: float) -> float: return lib().fo_fast_round_scale(a)


def act_quant_fp8(x, block: int = 32, round_scale: bool = True):
    x = _f32(x).ravel()
    y = np.empty(x.size, np.uint8)
    s = np.empty(x.size // block, np.float32)
    lib().fo_act_quant_fp8(_p(x), x.size, block, int(round_scale), _p(y), _p(s))
    return y, s


def act_quant_fp8_x2(x):
    """Two-term quantisation (block 32, power-of-two scales): (q1, s1, q2, s2) with x ~ dq1 + dq2."""
    x = _f32(x).ravel()
    q1, q2 = np.empty(x.size, np.uint8), np.empty(x.size, np.uint8)
    s1, s2 = np.empty(x.size // 32, np.float32), np.empty(x.size // 32, np.float32)
    lib().fo_act_quant_fp8_x2(_p(x), x.size, _p(q1), _p(s1), _p(q2), _p(s2))
    return q1, s1, q2, s2


def act_quant_fp4(x, block: int = 32, round_scale: bool = True):
    x = _f32(x).ravel()
    y = np.empty(x.size // 2, np.uint8)
    s = np.empty(x.size // block, np.float32)
    lib().fo_act_quant_fp4(_p(x), x.size, block, int(round_scale), _p(y), _p(s))
    return y, s


def dequant_fp4_row32(w, scale) -> np.ndarray:
    w, scale = _u8(w), _u8(scale)
    out, half = w.shape
    dst = np.empty((out, half * 2), np.float32)
    lib().fo_dequant_fp4_row32(_p(w), _p(scale), out, half * 2, _p(dst))
    return dst


# ---- CpuBackend ops ----
def matmul(x, w, bias=None) -> np.ndarray:
    x, w = _f32(x), _f32(w)
    n, k = x.shape
    o, k2 = w.shape
    if k != k2:
        raise OracleError("matmul: ShapeMismatch")
    b = None if bias is None else _f32(bias)
    out = np.empty((n, o), np.float32)
    _ck(lib().fo_matmul(_p(x), _p(w), _p(b), _p(out), n, k, o), "matmul")
    return out


def swiglu_limited(gate_up, limit: float) -> np.ndarray:
    g = _f32(gate_up)
    n, two_i = g.shape
    if two_i % 2:
        raise OracleError("swiglu last dim must be even")
    out = np.empty((n, two_i // 2), np.float32)
    _ck(lib().fo_swiglu_limited(_p(g), limit, _p(out), n, two_i // 2), "swiglu")
    return out


def rmsnorm(x, w, eps: float) -> np.ndarray:
    """cpu.rs:124-143; x [n, dim], w [dim]."""
    xv, wv = _f32(x), _f32(w)
    n, dim = xv.shape
    if wv.size != dim:
        raise OracleError("rmsnorm shape mismatch")
    out = np.empty_like(xv)
    _ck(lib().fo_rmsnorm(_p(xv), _p(wv), eps, _p(out), n, dim), "rmsnorm")
    return out


def hc_post(x, residual, post, comb) -> np.ndarray:
    """cpu.rs:788-807; x [s,h], residual [s,nh,h], post [s,nh], comb [s,nh,nh] -> [s,nh,h]."""
    xv, rv, pv, cv = _f32(x), _f32(residual), _f32(post), _f32(comb)
    s, h = xv.shape
    nh = rv.shape[1]
    if rv.shape != (s, nh, h) or pv.shape != (s, nh) or cv.shape != (s, nh, nh):
        raise OracleError("hc_post shape mismatch")
    out = np.empty_like(rv)
    _ck(lib().fo_hc_post(_p(xv), _p(rv), _p(pv), _p(cv), _p(out), s, nh, h), "hc_post")
    return out


def moe_route(logits, bias, topk: int, routed_scaling: float, n_group: int = 1, topk_group: int = 1,
              nan_policy: int = 0):
    """nan_policy 0: a NaN score raises (CpuBackend panics); 1: the reference's device router (never selected,
    unfillable slots get id -1 and weight 0)."""
    lg, b = _f32(logits), _f32(bias)
    n, e = lg.shape
    if b.size != e:
        raise OracleError("router bias shape")
    probs = np.empty((n, topk), np.float32)
    ids = np.empty((n, topk), np.float32)
    _ck(lib().fo_moe_route_grouped_nan(_p(lg), _p(b), n, e, topk, n_group, topk_group, routed_scaling, nan_policy,
                                       _p(probs), _p(ids)), "moe_route")
    return probs, ids


def expert_ffn(x, gate_w, up_w, down_w, limit: float) -> np.ndarray:
    x, gw, uw, dw = _f32(x), _f32(gate_w), _f32(up_w), _f32(down_w)
    m, h = x.shape
    inter = gw.shape[0]
    out = np.empty((m, h), np.float32)
    _ck(lib().fo_expert_ffn(_p(x), _p(gw), _p(uw), _p(dw), limit, _p(out), m, h, inter), "expert_ffn")
    return out


# ---- permutation ----
def moe_permute(ids, n_experts: int):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    n, topk = ids.shape
    counts = np.empty(n_experts, np.int32)
    starts = np.empty(n_experts + 1, np.int32)
    perm_map = np.empty(n * topk, np.int32)
    gather_src = np.empty(n * topk, np.int32)
    active = np.empty(n_experts, np.int32)
    n_active = np.zeros(1, np.int32)
    _ck(lib().fo_moe_permute(_p(ids), n, topk, n_experts, _p(counts), _p(starts), _p(perm_map),
                             _p(gather_src), _p(active), _p(n_active)), "moe_permute")
    return dict(counts=counts, starts=starts, perm_map=perm_map, gather_src=gather_src, active=active,
                n_active=int(n_active[0]))


def moe_align_host(idx: Sequence[int], topk: int, seg_cap: int, bm: int):
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    order = np.empty(seg_cap * bm, np.int32)
    counts = np.empty(seg_cap, np.int32)
    eid = np.empty(seg_cap, np.int32)
    nseg = lib().fo_moe_align_host(_p(idx), idx.size, topk, seg_cap, bm, _p(order), _p(counts), _p(eid))
    if nseg < 0:
        return None
    return order, counts, eid, nseg


# ---- the layer ----
def moe_ffn_mxfp4(inp, act_mode: int = 0, n_threads: int = 1, tok_sel=None, want_out: bool = True):
    """inp: ferrite_amd.synth.MoeInputs-like (cfg + numpy tensors).  Returns dict(out, logits, probs, ids)."""
    cfg = inp.cfg
    c = _Cfg(cfg.n, cfg.hidden, cfg.n_experts, cfg.topk, cfg.inter, cfg.shared_inter, cfg.n_group,
             cfg.topk_group, cfg.routed_scaling, cfg.swiglu_limit, act_mode, n_threads)
    keep = [_u8(getattr(inp, k)) for k in ("gate_w", "gate_s", "up_w", "up_s", "down_w", "down_s",
                                           "sh_gate_w", "sh_gate_s", "sh_up_w", "sh_up_s", "sh_down_w",
                                           "sh_down_s")]
    rw, rb = _f32(inp.router_w), _f32(inp.router_bias)
    w = _Weights(*[a.ctypes.data for a in keep], rw.ctypes.data, rb.ctypes.data)
    x = _f32(inp.x)
    sel = None if tok_sel is None else np.ascontiguousarray(tok_sel, dtype=np.int32)
    ns = cfg.n if sel is None else sel.size
    out = np.empty((ns, cfg.hidden), np.float32) if want_out else None
    logits = np.empty((cfg.n, cfg.n_experts), np.float32)
    probs = np.empty((cfg.n, cfg.topk), np.float32)
    ids = np.empty((cfg.n, cfg.topk), np.float32)
    _ck(lib().fo_moe_ffn_mxfp4(C.byref(c), C.byref(w), _p(x), _p(sel), ns, _p(out), _p(logits), _p(probs),
                               _p(ids)), "moe_ffn_mxfp4")
    return dict(out=out, logits=logits, probs=probs, ids=ids)
