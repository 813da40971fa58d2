"""Host-side mirror of the reference's kernel interface for the MoE FFN path, over libferrite_hip.so.

`HipBackend` has the methods of ferrite-kernel's `KernelBackend` that lie on the path (matmul, swiglu_limited,
moe_route: crates/ferrite-kernel/src/lib.rs:73,83-85,194-206), the `GraphCapable` capture/verify quartet
(crates/ferrite-kernel/src/graph.rs:48-64) and, like `CudaBackend::moe_layer_dev`
(crates/ferrite-kernel/src/cuda.rs:5604-6142), an inherent fused-layer entry `moe_layer_dev_mxfp4`.
Inputs are device tensors, outputs are pre-allocated by the caller, errors are raised as FerriteError
subclasses (never a crash), exactly as the reference returns `Err` for shape problems (cpu.rs:91-101,539-545).

torch is used for device memory and streams only.  There is no CPU fallback: if the shared library is missing
or no GPU is present the constructor raises.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass
from typing import Dict, List, Optional

import numpy as np
import torch

from .synth import MoeConfig, MoeInputs

_HERE = os.path.dirname(os.path.abspath(__file__))
DEFAULT_SO = os.path.join(_HERE, "libferrite_hip.so")
ABI_VERSION = 3

OK, ERR_INVALID_ARG, DECLINED, ERR_WORKSPACE, ERR_RUNTIME = 0, 1, 2, 3, 4
DT_F32, DT_BF16 = 0, 1
MODE_F32_CHECK, MODE_MFMA_FP8, MODE_MFMA_FP8_X2 = 0, 1, 2
OVERRIDE_UNIT_ROWS, OVERRIDE_Y_F32, OVERRIDE_PREFILL_TILE, OVERRIDE_HEAD = 0, 1, 2, 3


class FerriteError(RuntimeError):
    """crates/ferrite-types/src/lib.rs:143-159"""


class InvalidArg(FerriteError):
    pass


class ShapeMismatch(FerriteError):
    pass


class Declined(FerriteError):
    """The kernel declined the shape (the reference's callers fall back, cuda.rs:5763-5765)."""


class MoeShape(C.Structure):
    _fields_ = [("hidden", C.c_int), ("n_experts", C.c_int), ("topk", C.c_int), ("inter", C.c_int),
                ("shared_inter", C.c_int), ("n_group", C.c_int), ("topk_group", C.c_int),
                ("routed_scaling", C.c_float), ("swiglu_limit", C.c_float)]


_WEIGHT_FIELDS = ("router_w", "router_bias", "gate_w", "gate_s", "up_w", "up_s", "down_w", "down_s",
                  "sh_gate_w", "sh_gate_s", "sh_up_w", "sh_up_s", "sh_down_w", "sh_down_s")


class MoeWeights(C.Structure):
    _fields_ = [(k, C.c_void_p) for k in _WEIGHT_FIELDS]


STAGE_EVENTS = 10   # FERRITE_MOE_STAGE_EVENTS
STATIC_WORKSPACE_BYTES = 16 << 20   # FERRITE_STATIC_WORKSPACE_BYTES


class MoeExpertSrc(C.Structure):
    _fields_ = [(k, C.c_void_p) for k in ("gate_w", "gate_s", "up_w", "up_s", "down_w", "down_s")] + \
               [("gate_up_scale_pitch", C.c_int64), ("down_scale_pitch", C.c_int64)]


class MoeBlockArgs(C.Structure):
    _fields_ = [("norm_w", C.c_void_p), ("eps", C.c_float), ("residual", C.c_void_p), ("post", C.c_void_p),
                ("comb", C.c_void_p), ("nh", C.c_int)]


class WorkspaceView(C.Structure):
    _fields_ = [(k, C.c_void_p) for k in ("logits", "probs", "ids_f32", "ids", "counts", "starts", "perm_map",
                                          "gather_src", "active", "n_active", "y")]


EXPORTS = [
    "ferrite_kernel_build_id", "ferrite_kernel_abi_version", "ferrite_hip_last_error", "ferrite_hip_warmup",
    "ferrite_hip_set_override", "ferrite_matmul_f32", "ferrite_rmsnorm_f32", "ferrite_hc_post_f32",
    "ferrite_swiglu_limited_f32", "ferrite_moe_route", "ferrite_moe_permute_scratch_bytes", "ferrite_moe_permute",
    "ferrite_mxfp4_dequant", "ferrite_mxfp4_quant", "ferrite_act_quant_fp8", "ferrite_act_quant_fp8_x2",
    "ferrite_moe_packed_bytes",
    "ferrite_moe_pack_weights", "ferrite_moe_pack_expert", "ferrite_moe_pack_router",
    "ferrite_moe_packed_dequant", "ferrite_moe_layer_workspace_bytes", "ferrite_moe_layer_unit_rows", "ferrite_moe_block_workspace_bytes", "ferrite_moe_block_mxfp4", "ferrite_moe_layer_workspace_init", "ferrite_moe_layer_workspace_view",
    "ferrite_moe_layer_mxfp4", "ferrite_moe_layer_mxfp4_static", "ferrite_moe_layer_mxfp4_timed",
    "ferrite_moe_layer_check",
    "ferrite_graph_begin", "ferrite_graph_end", "ferrite_graph_launch",
    "ferrite_graph_destroy",
]


def load_library(so_path: Optional[str] = None) -> C.CDLL:
    """dlopen the library and run the identity checks the reference runs (cuda.rs:2061-2102)."""
    path = so_path or DEFAULT_SO
    if not os.path.exists(path):
        raise FerriteError(f"{path} not found: build it with `python -m ferrite_amd.build` (no CPU fallback exists)")
    lib = C.CDLL(path)
    vp, i32, f32, sz, i64 = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_int64
    lib.ferrite_kernel_build_id.restype = C.c_char_p
    lib.ferrite_kernel_abi_version.restype = C.c_uint
    lib.ferrite_hip_last_error.restype = C.c_char_p
    lib.ferrite_matmul_f32.argtypes = [vp, vp, vp, vp, i32, i32, i32, vp]
    lib.ferrite_swiglu_limited_f32.argtypes = [vp, f32, vp, i32, i32, vp]
    lib.ferrite_rmsnorm_f32.argtypes = [vp, vp, f32, vp, i32, i32, vp]
    lib.ferrite_hc_post_f32.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, vp]
    lib.ferrite_moe_route.argtypes = [vp, vp, i32, i32, i32, i32, i32, f32, vp, vp, vp, vp]
    lib.ferrite_moe_permute_scratch_bytes.restype = sz
    lib.ferrite_moe_permute_scratch_bytes.argtypes = [i32, i32, i32]
    lib.ferrite_hip_warmup.argtypes = []
    lib.ferrite_hip_set_override.argtypes = [i32, i32]
    lib.ferrite_moe_permute.argtypes = [vp, i32, i32, i32, vp, vp, vp, vp, vp, vp, vp, sz, vp]
    lib.ferrite_mxfp4_dequant.argtypes = [vp, vp, i64, i64, vp, vp]
    lib.ferrite_act_quant_fp8.argtypes = [vp, i32, i64, i32, vp, vp, vp]
    lib.ferrite_act_quant_fp8_x2.argtypes = [vp, i32, i64, i32, vp, vp, vp, vp, vp]
    lib.ferrite_mxfp4_quant.argtypes = [vp, i32, i64, i64, vp, vp, vp]
    lib.ferrite_moe_pack_expert.argtypes = [vp, i32, vp, vp, vp]
    lib.ferrite_moe_pack_router.argtypes = [vp, vp, vp, vp]
    lib.ferrite_moe_packed_bytes.restype = sz
    lib.ferrite_moe_packed_bytes.argtypes = [C.POINTER(MoeShape)]
    lib.ferrite_moe_pack_weights.argtypes = [C.POINTER(MoeShape), C.POINTER(MoeWeights), vp, vp]
    lib.ferrite_moe_packed_dequant.argtypes = [C.POINTER(MoeShape), vp, i32, i32, vp, vp]
    lib.ferrite_moe_layer_workspace_bytes.restype = sz
    lib.ferrite_moe_layer_unit_rows.argtypes = [C.POINTER(MoeShape), i32, i32]
    lib.ferrite_moe_block_workspace_bytes.restype = sz
    lib.ferrite_moe_block_workspace_bytes.argtypes = [C.POINTER(MoeShape), i32, i32]
    lib.ferrite_moe_block_mxfp4.argtypes = [C.POINTER(MoeShape), C.POINTER(MoeWeights), vp, vp, C.POINTER(MoeBlockArgs), i32,
                                            vp, i32, vp, sz, vp]
    lib.ferrite_moe_layer_workspace_bytes.argtypes = [C.POINTER(MoeShape), i32, i32]
    lib.ferrite_moe_layer_workspace_init.argtypes = [C.POINTER(MoeShape), i32, i32, vp, sz, vp]
    lib.ferrite_moe_layer_workspace_view.argtypes = [C.POINTER(MoeShape), i32, i32, vp, C.POINTER(WorkspaceView)]
    lib.ferrite_moe_layer_mxfp4.argtypes = [C.POINTER(MoeShape), C.POINTER(MoeWeights), vp, vp, i32, i32, vp, i32,
                                            i32, vp, sz, vp]
    lib.ferrite_moe_layer_mxfp4_timed.argtypes = lib.ferrite_moe_layer_mxfp4.argtypes + [C.POINTER(vp)]
    lib.ferrite_moe_layer_check.argtypes = [C.POINTER(MoeShape), i32, i32]
    lib.ferrite_moe_layer_mxfp4_static.argtypes = [C.POINTER(MoeShape), C.POINTER(MoeWeights), vp, vp, i32, i32, vp, i32,
                                                   i32, vp]
    lib.ferrite_graph_begin.argtypes = [vp]
    lib.ferrite_graph_end.argtypes = [vp, C.POINTER(vp)]
    lib.ferrite_graph_launch.argtypes = [vp, vp]
    lib.ferrite_graph_destroy.argtypes = [vp]
    if lib.ferrite_kernel_abi_version() != ABI_VERSION:
        raise FerriteError(f"ABI version {lib.ferrite_kernel_abi_version()} != {ABI_VERSION}")
    return lib


# ---- the op recorder of graph.rs:20-135 (host logic; identical state machine) ----
@dataclass(frozen=True)
class OpRecord:
    op: str
    shapes: tuple = ()


class OpTrace:
    def __init__(self, ops: Optional[List[OpRecord]] = None, graph_exec: Optional[int] = None):
        self.ops = list(ops or [])
        self.graph_exec = graph_exec

    def __len__(self):
        return len(self.ops)

    def is_empty(self):
        return not self.ops

    def __eq__(self, other):
        return isinstance(other, OpTrace) and self.ops == other.ops


class Recorder:
    OFF, CAPTURE, VERIFY = 0, 1, 2

    def __init__(self):
        self.mode = Recorder.OFF
        self.ops: List[OpRecord] = []
        self._trace: Optional[OpTrace] = None
        self._pos = 0
        self._ok = True

    def record(self, op: str, shapes=()):
        if self.mode == Recorder.CAPTURE:
            self.ops.append(OpRecord(op, tuple(map(tuple, shapes))))
        elif self.mode == Recorder.VERIFY and self._ok:
            rec = OpRecord(op, tuple(map(tuple, shapes)))
            if self._pos >= len(self._trace.ops) or self._trace.ops[self._pos] != rec:
                self._ok = False
            else:
                self._pos += 1

    def begin_capture(self):
        self.ops = []
        self.mode = Recorder.CAPTURE

    def end_capture(self) -> OpTrace:
        self.mode = Recorder.OFF
        ops, self.ops = self.ops, []
        return OpTrace(ops)

    def begin_verify(self, trace: OpTrace):
        self.mode, self._trace, self._pos, self._ok = Recorder.VERIFY, trace, 0, True

    def end_verify(self) -> bool:
        if self.mode != Recorder.VERIFY:
            self.mode = Recorder.OFF
            return False
        self.mode = Recorder.OFF
        return self._ok and self._pos == len(self._trace.ops)


def shape_of(cfg: MoeConfig) -> MoeShape:
    return MoeShape(cfg.hidden, cfg.n_experts, cfg.topk, cfg.inter, cfg.shared_inter, cfg.n_group,
                    cfg.topk_group, cfg.routed_scaling, cfg.swiglu_limit)


class MoeLayer:
    """Device-resident weights of one layer: checkpoint layout (optional) and the packed tile layout."""

    def __init__(self, cfg: MoeConfig, tensors: Dict[str, torch.Tensor], packed: Optional[torch.Tensor]):
        self.cfg = cfg
        self.shape = shape_of(cfg)
        self.tensors = tensors
        self.packed = packed
        self.weights = MoeWeights(*[(tensors[k].data_ptr() if k in tensors and tensors[k] is not None else None)
                                    for k in _WEIGHT_FIELDS])
        self._ws: Dict[tuple, torch.Tensor] = {}


class HipBackend:
    def __init__(self, so_path: Optional[str] = None, device: int = 0):
        self.lib = load_library(so_path)
        if not torch.cuda.is_available():
            raise FerriteError("no GPU visible: HipBackend has no CPU path")
        self.device = torch.device("cuda", device)
        torch.cuda.set_device(self.device)
        self.stream = torch.cuda.Stream(device=self.device)   # one stream per backend (cuda.rs:996)
        self.recorder = Recorder()
        self._capturing = False
        self._graphs: Dict[str, int] = {}
        self._verify_ok = False
        self._overrides = {OVERRIDE_UNIT_ROWS: 0, OVERRIDE_Y_F32: 0, OVERRIDE_PREFILL_TILE: 0, OVERRIDE_HEAD: 0}
        self._ck(self.lib.ferrite_hip_warmup(), "warmup")   # LDS limits, before any capture (cuda.rs:627-657)

    # ---- plumbing ----
    @property
    def build_id(self) -> str:
        return self.lib.ferrite_kernel_build_id().decode()

    def _st(self):
        return C.c_void_p(self.stream.cuda_stream)

    def _ck(self, rc: int, what: str):
        if rc == OK:
            return
        if rc == DECLINED:
            raise Declined(f"{what}: shape declined")
        if rc == ERR_RUNTIME:
            raise FerriteError(f"HIP {what}: {self.lib.ferrite_hip_last_error().decode()}")
        raise InvalidArg(f"{what}: rc={rc}")

    def _dev(self, t: torch.Tensor, dtype, what: str):
        if not isinstance(t, torch.Tensor) or t.device.type != "cuda":
            raise InvalidArg(f"{what} must be a device tensor")
        if t.dtype != dtype:
            raise InvalidArg(f"{what} dtype {t.dtype} != {dtype}")
        if not t.is_contiguous():
            raise InvalidArg(f"{what} must be contiguous")
        return t

    def _enter(self):
        """Make this backend's stream wait for work already queued on torch's current stream (not while a
        capture is open: the capture must stay on one stream)."""
        if not self._capturing:
            self.stream.wait_stream(torch.cuda.current_stream(self.device))

    def _leave(self):
        """Make torch's current stream wait for what was just enqueued, so torch ops on the outputs are ordered."""
        if not self._capturing:
            torch.cuda.current_stream(self.device).wait_stream(self.stream)

    def sync(self):
        self.stream.synchronize()

    def set_override(self, which: int, value: int):
        """Process-wide test hook of the library (token tile of the expert GEMMs, f32 expert outputs).  Changes the
        workspace layout: cached workspaces of a layer must be dropped by the caller (layer._ws.clear())."""
        self._ck(self.lib.ferrite_hip_set_override(which, value), "set_override")
        self._overrides[which] = value

    def upload(self, a, dtype=None) -> torch.Tensor:
        t = torch.from_numpy(np.ascontiguousarray(a))
        if dtype is not None:
            t = t.to(dtype)
        return t.to(self.device)

    # ---- KernelBackend ops on the path ----
    def matmul(self, x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor):
        """lib.rs:73 / cpu.rs:82-122 (recorded twice, like the reference: cpu.rs:89-90)."""
        self.recorder.record("matmul")
        self._leave()
        self.recorder.record("matmul")
        if x.dim() != 2 or w.dim() != 2:
            raise InvalidArg("matmul operands must be 2-d")
        n, k = x.shape
        o, k2 = w.shape
        if k != k2:
            raise ShapeMismatch(f"expected {tuple(x.shape)}, got {tuple(w.shape)}")
        if tuple(out.shape) != (n, o):
            raise InvalidArg(f"matmul out shape {tuple(out.shape)} != [{n},{o}]")
        self._dev(x, torch.float32, "x"); self._dev(w, torch.float32, "w"); self._dev(out, torch.float32, "out")
        if bias is not None:
            self._dev(bias, torch.float32, "bias")
            if bias.numel() != o:
                raise InvalidArg("matmul bias shape")
        self._enter()
        self._ck(self.lib.ferrite_matmul_f32(x.data_ptr(), w.data_ptr(), None if bias is None else bias.data_ptr(),
                                             out.data_ptr(), n, k, o, self._st()), "matmul")

    def rmsnorm(self, x: torch.Tensor, w: torch.Tensor, eps: float, out: torch.Tensor):
        """lib.rs:76 / cpu.rs:124-143: x, out [..., dim] f32, w [dim] f32."""
        self.recorder.record("rmsnorm")
        self._leave()
        if x.dim() < 1:
            raise InvalidArg("rmsnorm rank 0")
        dim = x.shape[-1]
        if w.numel() != dim or tuple(out.shape) != tuple(x.shape):
            raise InvalidArg("rmsnorm shape mismatch")
        self._dev(x, torch.float32, "x"); self._dev(w, torch.float32, "w"); self._dev(out, torch.float32, "out")
        self._enter()
        self._ck(self.lib.ferrite_rmsnorm_f32(x.data_ptr(), w.data_ptr(), eps, out.data_ptr(), x.numel() // dim, dim,
                                              self._st()), "rmsnorm")

    def hc_post(self, x: torch.Tensor, residual: torch.Tensor, post: torch.Tensor, comb: torch.Tensor) -> torch.Tensor:
        """lib.rs:256 / cpu.rs:788-807: x [s,h], residual [s,nh,h], post [s,nh], comb [s,nh,nh] -> new [s,nh,h]."""
        self.recorder.record("hc_post")
        self._leave()
        if x.dim() != 2 or residual.dim() != 3:
            raise InvalidArg("hc_post expects x [s,h] and residual [s,nh,h]")
        s, h = x.shape
        nh = residual.shape[1]
        if tuple(residual.shape) != (s, nh, h) or tuple(post.shape) != (s, nh) or tuple(comb.shape) != (s, nh, nh):
            raise ShapeMismatch("hc_post shape mismatch")
        for t, nm in ((x, "x"), (residual, "residual"), (post, "post"), (comb, "comb")):
            self._dev(t, torch.float32, nm)
        out = torch.empty_like(residual)
        self._enter()
        self._ck(self.lib.ferrite_hc_post_f32(x.data_ptr(), residual.data_ptr(), post.data_ptr(), comb.data_ptr(),
                                              out.data_ptr(), s, nh, h, self._st()), "hc_post")
        return out

    def swiglu_limited(self, gate_up: torch.Tensor, limit: float, out: torch.Tensor):
        """lib.rs:83-85 / cpu.rs:178-203"""
        self.recorder.record("swiglu")
        self._leave()
        if gate_up.dim() != 2:
            raise InvalidArg("swiglu input must be 2-d")
        n, two_i = gate_up.shape
        if two_i % 2:
            raise InvalidArg("swiglu last dim must be even")
        if tuple(out.shape) != (n, two_i // 2):
            raise InvalidArg(f"swiglu out {tuple(out.shape)} != [{n},{two_i // 2}]")
        self._dev(gate_up, torch.float32, "gate_up"); self._dev(out, torch.float32, "out")
        self._enter()
        self._ck(self.lib.ferrite_swiglu_limited_f32(gate_up.data_ptr(), limit, out.data_ptr(), n, two_i // 2,
                                                     self._st()), "swiglu")

    def moe_route(self, logits: torch.Tensor, bias: torch.Tensor, topk: int, routed_scaling: float,
                  probs: torch.Tensor, ids: torch.Tensor, n_group: int = 1, topk_group: int = 1,
                  ids_i32: Optional[torch.Tensor] = None):
        """lib.rs:194-206 / cpu.rs:528-572; ids is an f32 tensor as in the reference."""
        self.recorder.record("moe_route")
        self._leave()
        self.recorder.record("moe_route")
        if logits.dim() != 2:
            raise InvalidArg("logits must be 2-d")
        n, e = logits.shape
        if bias.numel() != e:
            raise InvalidArg("router bias shape")
        if tuple(probs.shape) != (n, topk) or tuple(ids.shape) != (n, topk):
            raise InvalidArg("router out shape")
        self._dev(logits, torch.float32, "logits"); self._dev(bias, torch.float32, "bias")
        self._dev(probs, torch.float32, "probs"); self._dev(ids, torch.float32, "ids")
        if ids_i32 is not None:
            self._dev(ids_i32, torch.int32, "ids_i32")
        self._enter()
        self._ck(self.lib.ferrite_moe_route(logits.data_ptr(), bias.data_ptr(), n, e, topk, n_group, topk_group,
                                            routed_scaling, probs.data_ptr(), ids.data_ptr(),
                                            None if ids_i32 is None else ids_i32.data_ptr(), self._st()), "moe_route")

    # ---- inherent ops ----
    def moe_permute(self, ids: torch.Tensor, n_experts: int) -> Dict[str, torch.Tensor]:
        self.recorder.record("moe_permute")
        self._dev(ids, torch.int32, "ids")
        if ids.dim() != 2:
            raise InvalidArg("ids must be [n, topk]")
        n, topk = ids.shape
        mk = lambda m: torch.empty(m, dtype=torch.int32, device=self.device)
        t = dict(counts=mk(n_experts), starts=mk(n_experts + 1), perm_map=mk(n * topk), gather_src=mk(n * topk),
                 active=mk(n_experts), n_active=mk(1))
        sb = self.lib.ferrite_moe_permute_scratch_bytes(n, topk, n_experts)
        scratch = torch.empty(max(sb, 16), dtype=torch.uint8, device=self.device)
        self._enter()
        self._ck(self.lib.ferrite_moe_permute(ids.data_ptr(), n, topk, n_experts, t["counts"].data_ptr(),
                                              t["starts"].data_ptr(), t["perm_map"].data_ptr(),
                                              t["gather_src"].data_ptr(), t["active"].data_ptr(),
                                              t["n_active"].data_ptr(), scratch.data_ptr(), sb, self._st()),
                 "moe_permute")
        self.sync()   # scratch goes out of scope
        return t

    def mxfp4_dequant(self, w: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
        self._dev(w, torch.uint8, "w"); self._dev(scale, torch.uint8, "scale")
        rows = w.numel() // w.shape[-1]
        cols = w.shape[-1] * 2
        if scale.numel() != rows * (cols // 32):
            raise ShapeMismatch("scale shape")
        out = torch.empty(tuple(w.shape[:-1]) + (cols,), dtype=torch.float32, device=self.device)
        self._enter()
        self._ck(self.lib.ferrite_mxfp4_dequant(w.data_ptr(), scale.data_ptr(), rows, cols, out.data_ptr(),
                                                self._st()), "mxfp4_dequant")
        self._leave()
        return out

    def mxfp4_quant(self, x: torch.Tensor):
        """[rows, cols] f32 / bf16 -> (codes [rows, cols/2] u8, scales [rows, cols/32] u8), quant.rs:217-238."""
        if x.dtype not in (torch.float32, torch.bfloat16) or x.dim() != 2 or not x.is_contiguous():
            raise InvalidArg("x must be contiguous [rows, cols] f32 or bf16")
        rows, cols = x.shape
        if cols % 32:
            raise InvalidArg("cols must be a multiple of 32")
        self._dev(x, x.dtype, "x")
        codes = torch.empty((rows, cols // 2), dtype=torch.uint8, device=self.device)
        s = torch.empty((rows, cols // 32), dtype=torch.uint8, device=self.device)
        self._enter()
        self._ck(self.lib.ferrite_mxfp4_quant(x.data_ptr(), DT_F32 if x.dtype == torch.float32 else DT_BF16, rows,
                                              cols, codes.data_ptr(), s.data_ptr(), self._st()), "mxfp4_quant")
        self._leave()
        return codes, s

    def pack_expert(self, layer: MoeLayer, expert: int, gate=None, up=None, down=None, gate_up_scale_pitch: int = 0,
                    down_scale_pitch: int = 0):
        """Repack one expert's matrices into layer.packed: gate / up / down are (codes, scales) pairs of device
        uint8 tensors in the checkpoint layout, or None to leave that group as it is."""
        src = MoeExpertSrc()
        keep = []
        for key, pair in (("gate", gate), ("up", up), ("down", down)):
            if pair is None:
                continue
            w, s = pair
            self._dev(w, torch.uint8, key + " codes"); self._dev(s, torch.uint8, key + " scales")
            setattr(src, key + "_w", w.data_ptr()); setattr(src, key + "_s", s.data_ptr())
            keep += [w, s]
        src.gate_up_scale_pitch, src.down_scale_pitch = gate_up_scale_pitch, down_scale_pitch
        self._enter()
        self._ck(self.lib.ferrite_moe_pack_expert(C.byref(layer.shape), expert, C.byref(src), layer.packed.data_ptr(),
                                                  self._st()), "pack_expert")
        self._leave()

    def act_quant_fp8(self, x: torch.Tensor):
        if x.dtype not in (torch.float32, torch.bfloat16) or x.dim() != 2 or not x.is_contiguous():
            raise InvalidArg("x must be contiguous [rows, cols] f32 or bf16")
        rows, cols = x.shape
        if cols % 32:
            raise InvalidArg("cols must be a multiple of 32")
        q = torch.empty((rows, cols), dtype=torch.uint8, device=self.device)
        s = torch.empty((rows, cols // 32), dtype=torch.uint8, device=self.device)
        self._enter()
        self._ck(self.lib.ferrite_act_quant_fp8(x.data_ptr(), DT_F32 if x.dtype == torch.float32 else DT_BF16, rows,
                                                cols, q.data_ptr(), s.data_ptr(), self._st()), "act_quant_fp8")
        self._leave()
        return q, s

    def act_quant_fp8_x2(self, x: torch.Tensor):
        """Two-term e4m3-per-32 quantisation: (q1, s1, q2, s2), the second pair from the residual of the first."""
        if x.dtype not in (torch.float32, torch.bfloat16) or x.dim() != 2 or not x.is_contiguous():
            raise InvalidArg("x must be contiguous [rows, cols] f32 or bf16")
        rows, cols = x.shape
        if cols % 32:
            raise InvalidArg("cols must be a multiple of 32")
        mk = lambda c: torch.empty((rows, c), dtype=torch.uint8, device=self.device)
        q1, s1, q2, s2 = mk(cols), mk(cols // 32), mk(cols), mk(cols // 32)
        self._enter()
        self._ck(self.lib.ferrite_act_quant_fp8_x2(x.data_ptr(), DT_F32 if x.dtype == torch.float32 else DT_BF16, rows,
                                                   cols, q1.data_ptr(), s1.data_ptr(), q2.data_ptr(), s2.data_ptr(),
                                                   self._st()), "act_quant_fp8_x2")
        self._leave()
        return q1, s1, q2, s2

    # ---- the fused layer ----
    def load_moe_layer(self, inp: MoeInputs, keep_checkpoint_layout: bool = True, pack: bool = True) -> MoeLayer:
        """Upload one layer's weights (checkpoint layout) and build the packed tile layout on the device."""
        cfg = inp.cfg
        tensors = {k: self.upload(getattr(inp, k)) for k in _WEIGHT_FIELDS}
        layer = MoeLayer(cfg, tensors, None)
        if pack:
            nbytes = self.lib.ferrite_moe_packed_bytes(C.byref(layer.shape))
            if nbytes == 0:
                raise Declined("shape not supported by the MFMA path")
            layer.packed = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
            self._enter()
            self._ck(self.lib.ferrite_moe_pack_weights(C.byref(layer.shape), C.byref(layer.weights),
                                                       layer.packed.data_ptr(), self._st()), "pack_weights")
            self.sync()
        if not keep_checkpoint_layout:
            for k in _WEIGHT_FIELDS[2:]:
                tensors[k] = None
            layer.weights = MoeWeights(*[(tensors[k].data_ptr() if tensors[k] is not None else None)
                                         for k in _WEIGHT_FIELDS])
        return layer

    def packed_dequant(self, layer: MoeLayer, expert: int, which: int) -> torch.Tensor:
        cfg = layer.cfg
        inter = cfg.shared_inter if expert == cfg.n_experts else cfg.inter
        rows, cols = (cfg.hidden, inter) if which == 2 else (inter, cfg.hidden)
        out = torch.empty((rows, cols), dtype=torch.float32, device=self.device)
        self._enter()
        self._ck(self.lib.ferrite_moe_packed_dequant(C.byref(layer.shape), layer.packed.data_ptr(), expert, which,
                                                     out.data_ptr(), self._st()), "packed_dequant")
        self._leave()
        return out

    def effective_mode(self, layer: MoeLayer, n: int, mode: int) -> int:
        """The mode a layer call for n tokens runs in: the one asked for, or, where the library declines it, the mode
        the caller falls back to (cuda.rs:5763-5765: a declined fused kernel is not an error, the other path runs).
        The order is two-term MFMA -> one-term MFMA -> the f32 mode; the MFMA modes decline shapes whose hidden or
        intermediate size is not a multiple of 128, which the f32 mode serves from the checkpoint-layout weights."""
        chain = [MODE_MFMA_FP8_X2, MODE_MFMA_FP8, MODE_F32_CHECK]
        if mode not in chain:
            return mode
        for m in chain[chain.index(mode):]:
            rc = self.lib.ferrite_moe_layer_check(C.byref(layer.shape), n, m)
            if rc == OK:
                return m
            if rc != DECLINED:
                break
        return mode

    def workspace(self, layer: MoeLayer, n: int, mode: int) -> torch.Tensor:
        mode = self.effective_mode(layer, n, mode)
        key = (n, mode)
        if key not in layer._ws:
            nbytes = self.lib.ferrite_moe_layer_workspace_bytes(C.byref(layer.shape), n, mode)
            if nbytes == 0:
                raise InvalidArg("unsupported shape / mode")
            ws = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
            self._enter()
            self._ck(self.lib.ferrite_moe_layer_workspace_init(C.byref(layer.shape), n, mode, ws.data_ptr(), nbytes,
                                                               self._st()), "workspace_init")
            self._leave()
            layer._ws[key] = ws
        return layer._ws[key]

    def unit_rows(self, layer: MoeLayer, n: int, mode: int = MODE_MFMA_FP8) -> int:
        """Token tile of the expert GEMMs for such a call: 16 (streaming kernels), or the tiled kernels' 128 (one-term
        activations) / 64 (two-term)."""
        return int(self.lib.ferrite_moe_layer_unit_rows(C.byref(layer.shape), n, self.effective_mode(layer, n, mode)))

    def moe_layer_dev_mxfp4(self, layer: MoeLayer, x: torch.Tensor, out: torch.Tensor, mode: int = MODE_MFMA_FP8,
                            workspace: Optional[torch.Tensor] = None, stage_events=None):
        """The whole layer on the device: router GEMM -> route -> permute -> experts -> combine (+shared).
        x [n, H] f32 or bf16, out [n, H] f32 or bf16, both pre-allocated device tensors."""
        self.recorder.record("moe_layer_mxfp4")
        self._leave()
        cfg = layer.cfg
        if x.dim() != 2 or x.shape[1] != cfg.hidden:
            raise ShapeMismatch(f"x {tuple(x.shape)} vs hidden {cfg.hidden}")
        n = x.shape[0]
        if tuple(out.shape) != (n, cfg.hidden):
            raise InvalidArg(f"out shape {tuple(out.shape)} != [{n},{cfg.hidden}]")
        dts = {torch.float32: DT_F32, torch.bfloat16: DT_BF16}
        if x.dtype not in dts or out.dtype not in dts or not x.is_contiguous() or not out.is_contiguous():
            raise InvalidArg("x/out must be contiguous f32 or bf16 device tensors")
        mode = self.effective_mode(layer, n, mode)   # a declined mode falls back, it is not an error
        if mode != MODE_F32_CHECK and layer.packed is None:
            raise InvalidArg("layer has no packed weights")
        ws = workspace if workspace is not None else self.workspace(layer, n, mode)
        self._enter()
        args = (C.byref(layer.shape), C.byref(layer.weights), None if layer.packed is None else layer.packed.data_ptr(),
                x.data_ptr(), dts[x.dtype], n, out.data_ptr(), dts[out.dtype], mode, ws.data_ptr(), ws.numel(),
                self._st())
        if stage_events is None:
            self._ck(self.lib.ferrite_moe_layer_mxfp4(*args), "moe_layer_mxfp4")
        else:
            if len(stage_events) != STAGE_EVENTS:
                raise InvalidArg(f"stage_events must hold {STAGE_EVENTS} event handles")
            self._ck(self.lib.ferrite_moe_layer_mxfp4_timed(*args, stage_events), "moe_layer_mxfp4")

    def moe_layer_dev_mxfp4_static(self, layer: MoeLayer, x: torch.Tensor, out: torch.Tensor, mode: int = MODE_MFMA_FP8):
        """The same layer on the library's built-in workspace: nothing is allocated, here or in the library."""
        self.recorder.record("moe_layer_mxfp4")
        self._leave()
        cfg = layer.cfg
        if x.dim() != 2 or x.shape[1] != cfg.hidden:
            raise ShapeMismatch(f"x {tuple(x.shape)} vs hidden {cfg.hidden}")
        n = x.shape[0]
        if tuple(out.shape) != (n, cfg.hidden):
            raise InvalidArg(f"out shape {tuple(out.shape)} != [{n},{cfg.hidden}]")
        dts = {torch.float32: DT_F32, torch.bfloat16: DT_BF16}
        if x.dtype not in dts or out.dtype not in dts or not x.is_contiguous() or not out.is_contiguous():
            raise InvalidArg("x/out must be contiguous f32 or bf16 device tensors")
        self._enter()
        rc = self.lib.ferrite_moe_layer_mxfp4_static(
            C.byref(layer.shape), C.byref(layer.weights), None if layer.packed is None else layer.packed.data_ptr(),
            x.data_ptr(), dts[x.dtype], n, out.data_ptr(), dts[out.dtype], mode, self._st())
        if rc == ERR_WORKSPACE:
            raise FerriteError(self.lib.ferrite_hip_last_error().decode())
        self._ck(rc, "moe_layer_mxfp4_static")

    def block_workspace(self, layer: MoeLayer, n: int, mode: int) -> torch.Tensor:
        mode = self.effective_mode(layer, n, mode)
        key = ("block", n, mode)
        if key not in layer._ws:
            nbytes = self.lib.ferrite_moe_block_workspace_bytes(C.byref(layer.shape), n, mode)
            if nbytes == 0:
                raise InvalidArg("unsupported shape / mode")
            ws = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
            self._enter()
            self._ck(self.lib.ferrite_moe_layer_workspace_init(C.byref(layer.shape), n, mode, ws.data_ptr(), nbytes,
                                                               self._st()), "workspace_init")
            self._leave()
            layer._ws[key] = ws
        return layer._ws[key]

    def moe_block_mxfp4(self, layer: MoeLayer, li: torch.Tensor, norm_w: torch.Tensor, eps: float,
                        residual: Optional[torch.Tensor], post: Optional[torch.Tensor], comb: Optional[torch.Tensor],
                        out: torch.Tensor, mode: int = MODE_MFMA_FP8, workspace: Optional[torch.Tensor] = None):
        """The FFN half of a decoder layer (exec/lib.rs:487-492): rmsnorm -> MoE FFN -> hc_post, one call.
        li [n,H] f32, residual/out [n,nh,H] f32, post [n,nh], comb [n,nh,nh].  residual None: rmsnorm -> MoE FFN
        only, out [n,H]."""
        self.recorder.record("moe_block_mxfp4")
        self._leave()
        cfg = layer.cfg
        if li.dim() != 2 or li.shape[1] != cfg.hidden:
            raise ShapeMismatch(f"li {tuple(li.shape)} vs hidden {cfg.hidden}")
        n = li.shape[0]
        tensors = [(li, "li"), (norm_w, "norm_w"), (out, "out")]
        if residual is None:
            nh = 0
            if tuple(out.shape) != (n, cfg.hidden) or norm_w.numel() != cfg.hidden:
                raise ShapeMismatch("moe_block shape mismatch")
        else:
            nh = residual.shape[1] if residual.dim() == 3 else -1
            if (tuple(residual.shape) != (n, nh, cfg.hidden) or tuple(out.shape) != (n, nh, cfg.hidden)
                    or tuple(post.shape) != (n, nh) or tuple(comb.shape) != (n, nh, nh) or norm_w.numel() != cfg.hidden):
                raise ShapeMismatch("moe_block shape mismatch")
            tensors += [(residual, "residual"), (post, "post"), (comb, "comb")]
        for t, nm in tensors:
            self._dev(t, torch.float32, nm)
        if mode != MODE_F32_CHECK and layer.packed is None:
            raise InvalidArg("layer has no packed weights")
        mode = self.effective_mode(layer, n, mode)
        ws = workspace if workspace is not None else self.block_workspace(layer, n, mode)
        ptr = lambda t: None if t is None else t.data_ptr()
        blk = MoeBlockArgs(norm_w.data_ptr(), eps, ptr(residual), ptr(post), ptr(comb), nh)
        self._enter()
        self._ck(self.lib.ferrite_moe_block_mxfp4(C.byref(layer.shape), C.byref(layer.weights),
                                                  None if layer.packed is None else layer.packed.data_ptr(),
                                                  li.data_ptr(), C.byref(blk), n, out.data_ptr(), mode, ws.data_ptr(),
                                                  ws.numel(), self._st()), "moe_block_mxfp4")

    def workspace_view(self, layer: MoeLayer, n: int, mode: int,
                       workspace: Optional[torch.Tensor] = None) -> Dict[str, torch.Tensor]:
        """Typed views of the intermediates the last layer call left in its workspace."""
        mode = self.effective_mode(layer, n, mode)
        ws = workspace if workspace is not None else self.workspace(layer, n, mode)
        v = WorkspaceView()
        self._ck(self.lib.ferrite_moe_layer_workspace_view(C.byref(layer.shape), n, mode, ws.data_ptr(), C.byref(v)),
                 "workspace_view")
        cfg = layer.cfg
        base = ws.data_ptr()
        rows = n * cfg.topk + (n if cfg.shared_inter > 0 else 0)

        def view(ptr, count, dtype):
            off = ptr - base
            size = torch.empty((), dtype=dtype).element_size()
            return ws[off:off + count * size].view(dtype)

        E, k = cfg.n_experts, cfg.topk
        y_bf16 = (mode != MODE_F32_CHECK and self.unit_rows(layer, n, mode) >= 64
                  and not self._overrides[OVERRIDE_Y_F32])
        y_dtype = torch.bfloat16 if y_bf16 else torch.float32
        return dict(logits=view(v.logits, n * E, torch.float32).view(n, E),
                    probs=view(v.probs, n * k, torch.float32).view(n, k),
                    ids_f32=view(v.ids_f32, n * k, torch.float32).view(n, k),
                    ids=view(v.ids, n * k, torch.int32).view(n, k),
                    counts=view(v.counts, E, torch.int32), starts=view(v.starts, E + 1, torch.int32),
                    perm_map=view(v.perm_map, n * k, torch.int32), gather_src=view(v.gather_src, n * k, torch.int32),
                    active=view(v.active, E, torch.int32), n_active=view(v.n_active, 1, torch.int32),
                    y=view(v.y, rows * cfg.hidden, y_dtype).view(rows, cfg.hidden))

    # ---- GraphCapable (graph.rs:48-64; device semantics of cuda.rs:3043-3092) ----
    def begin_capture(self):
        """Start stream capture; ops issued until end_capture are recorded into a graph, not executed."""
        self.recorder.begin_capture()
        self._enter()
        self._ck(self.lib.ferrite_graph_begin(self._st()), "graph_begin")
        self._capturing = True

    def end_capture(self) -> OpTrace:
        """End capture and instantiate.  The returned trace carries the op names and the graph handle."""
        exec_ = C.c_void_p()
        self._capturing = False
        rc = self.lib.ferrite_graph_end(self._st(), C.byref(exec_))
        trace = self.recorder.end_capture()
        if rc != OK:
            raise FerriteError(f"graph capture failed: {self.lib.ferrite_hip_last_error().decode()}")
        trace.graph_exec = exec_.value
        return trace

    def begin_verify(self, trace: OpTrace):
        """Replay launch of the captured graph into the same static buffers."""
        if trace.graph_exec is None:
            raise InvalidArg("trace holds no graph")
        self._enter()
        rc = self.lib.ferrite_graph_launch(C.c_void_p(trace.graph_exec), self._st())
        self._verify_ok = rc == OK

    def end_verify(self) -> bool:
        """True when the replay ran to completion."""
        try:
            self.sync()
        except RuntimeError:
            return False
        return self._verify_ok

    def graph_destroy(self, trace: OpTrace):
        if trace.graph_exec is not None:
            self.lib.ferrite_graph_destroy(C.c_void_p(trace.graph_exec))
            trace.graph_exec = None
