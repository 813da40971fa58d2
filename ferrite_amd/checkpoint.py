"""Checkpoint -> device for one MoE layer, over the C++ host library (libferrite_host.so).

The reader and the loader themselves are C++ (ferrite_amd/host/checkpoint.cpp), standing where the reference's
Rust loader does (crates/ferrite-models/src/dsv41/weights.rs:814-905 SafetensorsIndex / TensorView; names
:333-354 and crates/ferrite-model/src/weights.rs:133-149).  This module binds them with ctypes and adds a writer of
safetensors files for synthetic checkpoints (tests and the load benchmark have no real one to read).
"""
from __future__ import annotations

import ctypes as C
import json
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, List, Optional, Tuple

import numpy as np
import torch

from .backend import DEFAULT_SO, FerriteError, HipBackend, InvalidArg, MoeConfig, MoeLayer, MoeShape, shape_of

HOST_SO = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host", "libferrite_host.so")
NAMING_DSV41, NAMING_GLM = 0, 1
HOST_EXPORTS = ["ferrite_ckpt_open", "ferrite_ckpt_add_shard", "ferrite_ckpt_close", "ferrite_ckpt_num_tensors", "ferrite_ckpt_data_start",
                "ferrite_ckpt_tensor", "ferrite_ckpt_validate_moe", "ferrite_ckpt_load_moe_layer"]


def load_host_library(so_path: Optional[str] = None) -> C.CDLL:
    path = so_path or HOST_SO
    if not os.path.exists(path):
        raise FerriteError(f"{path} not found: build it with `python -m ferrite_amd.build`")
    lib = C.CDLL(path)
    vp, i32, sz, cp = C.c_void_p, C.c_int, C.c_size_t, C.c_char_p
    lib.ferrite_ckpt_open.restype = vp
    lib.ferrite_ckpt_open.argtypes = [cp, cp, sz]
    lib.ferrite_ckpt_add_shard.argtypes = [vp, cp, cp, sz]
    lib.ferrite_ckpt_close.restype = None
    lib.ferrite_ckpt_close.argtypes = [vp]
    lib.ferrite_ckpt_num_tensors.restype = C.c_int64
    lib.ferrite_ckpt_num_tensors.argtypes = [vp]
    lib.ferrite_ckpt_data_start.restype = C.c_uint64
    lib.ferrite_ckpt_data_start.argtypes = [vp]
    lib.ferrite_ckpt_tensor.argtypes = [vp, cp, cp, C.POINTER(C.c_int64), C.POINTER(i32), C.POINTER(C.c_uint64),
                                        C.POINTER(C.c_uint64)]
    lib.ferrite_ckpt_validate_moe.argtypes = [vp, i32, cp, C.POINTER(MoeShape), cp, sz]
    lib.ferrite_ckpt_load_moe_layer.argtypes = [vp, cp, i32, i32, cp, C.POINTER(MoeShape), vp, vp, i32, i32,
                                                C.POINTER(C.c_double), cp, sz]
    return lib


@dataclass
class TensorView:
    """weights.rs:814-823: dtype, shape and the byte range inside the data section."""
    dtype: str
    shape: Tuple[int, ...]
    begin: int
    end: int


@dataclass
class LoadStats:
    source_bytes: int
    packed_bytes: int
    seconds: float
    workers: int


class Checkpoint:
    """An opened checkpoint: one safetensors file, or the shards of a split one (header indexes + read-only
    mappings; a tensor is taken from the first shard that names it)."""

    def __init__(self, path, host_so: Optional[str] = None):
        paths = [path] if isinstance(path, (str, bytes, os.PathLike)) else list(path)
        if not paths:
            raise InvalidArg("no checkpoint file given")
        self.lib = load_host_library(host_so)
        self._h = None
        err = C.create_string_buffer(512)
        self._h = self.lib.ferrite_ckpt_open(os.fsencode(paths[0]), err, len(err))
        if not self._h:
            raise InvalidArg(err.value.decode(errors="replace"))
        for p in paths[1:]:
            if self.lib.ferrite_ckpt_add_shard(self._h, os.fsencode(p), err, len(err)) != 0:
                msg = err.value.decode(errors="replace")
                self.close()
                raise InvalidArg(msg)
        self.path = paths[0]
        self.paths = paths

    def close(self):
        if self._h:
            self.lib.ferrite_ckpt_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __len__(self) -> int:
        return int(self.lib.ferrite_ckpt_num_tensors(self._h))

    @property
    def data_start(self) -> int:
        return int(self.lib.ferrite_ckpt_data_start(self._h))

    def tensor(self, name: str) -> Optional[TensorView]:
        dt = C.create_string_buffer(16)
        shape = (C.c_int64 * 8)()
        ndim, b, e = C.c_int(0), C.c_uint64(0), C.c_uint64(0)
        rc = self.lib.ferrite_ckpt_tensor(self._h, name.encode(), dt, shape, C.byref(ndim), C.byref(b), C.byref(e))
        if rc != 0:
            return None
        return TensorView(dt.value.decode(), tuple(int(shape[i]) for i in range(min(ndim.value, 8))), b.value, e.value)

    def validate_moe(self, cfg: MoeConfig, prefix: str, naming: int) -> List[str]:
        """Missing names and shape mismatches of one layer's MoE tensors (weights.rs:882-905)."""
        shape = shape_of(cfg)
        report = C.create_string_buffer(1 << 16)
        n = self.lib.ferrite_ckpt_validate_moe(self._h, naming, prefix.encode(), C.byref(shape), report, len(report))
        if n < 0:
            raise InvalidArg("validate_moe: bad argument")
        return [ln for ln in report.value.decode().split("\n") if ln]

    def load_moe_layer(self, be: HipBackend, cfg: MoeConfig, prefix: str, naming: int, workers: int = 8,
                       pad_scale_rows: bool = False, hip_so: Optional[str] = None) -> Tuple[MoeLayer, LoadStats]:
        """Stream the layer into a packed device buffer; the returned layer holds `packed` and the routing bias
        only (no checkpoint-layout copy stays on the device)."""
        shape = shape_of(cfg)
        nbytes = be.lib.ferrite_moe_packed_bytes(C.byref(shape))
        if nbytes == 0:
            raise InvalidArg("shape not supported by the MFMA path")
        packed = torch.empty(nbytes, dtype=torch.uint8, device=be.device)
        bias = torch.zeros(cfg.n_experts, dtype=torch.float32, device=be.device)
        torch.cuda.synchronize(be.device)
        stats = (C.c_double * 4)()
        err = C.create_string_buffer(1024)
        rc = self.lib.ferrite_ckpt_load_moe_layer(self._h, os.fsencode(hip_so or DEFAULT_SO), be.device.index or 0,
                                                  naming, prefix.encode(), C.byref(shape), packed.data_ptr(),
                                                  bias.data_ptr(), workers, int(pad_scale_rows), stats, err, len(err))
        if rc != 0:
            raise InvalidArg(err.value.decode(errors="replace"))
        layer = MoeLayer(cfg, {"router_bias": bias}, packed)
        return layer, LoadStats(int(stats[0]), int(stats[1]), float(stats[2]), int(stats[3]))


# ---- writing synthetic checkpoints --------------------------------------------------------------------------

_NP_DTYPES = {"F32": np.float32, "I8": np.int8, "U8": np.uint8, "F8_E8M0": np.uint8, "F8_E4M3": np.uint8,
              "BF16": np.uint16, "I32": np.int32, "I64": np.int64, "F16": np.float16}


def write_safetensors(path: str, tensors: Iterable[Tuple[str, str, np.ndarray]],
                      metadata: Optional[Dict[str, str]] = None) -> None:
    """Write (name, dtype tag, array) triples as one safetensors file: 8-byte little-endian header length, the
    JSON header (padded with spaces to a multiple of 8), then the tensors' bytes back to back in the given order.
    The array's bytes are written as they are; the tag names how a reader interprets them (an e8m0 plane is a
    uint8 array tagged F8_E8M0, bf16 is a uint16 array tagged BF16)."""
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = metadata
    blobs, off = [], 0
    for name, tag, arr in tensors:
        if tag not in _NP_DTYPES:
            raise InvalidArg(f"dtype tag {tag}")
        a = np.ascontiguousarray(arr)
        if a.dtype.itemsize != np.dtype(_NP_DTYPES[tag]).itemsize:
            raise InvalidArg(f"{name}: array of {a.dtype} under tag {tag}")
        header[name] = {"dtype": tag, "shape": list(a.shape), "data_offsets": [off, off + a.nbytes]}
        blobs.append(a)
        off += a.nbytes
    js = json.dumps(header, separators=(",", ":")).encode()
    js += b" " * (-len(js) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(js)))
        f.write(js)
        for a in blobs:
            f.write(memoryview(a).cast("B"))


def moe_tensor_names(naming: int, prefix: str, expert: int, n_experts: int) -> Dict[str, str]:
    """The tensor-name stems of one expert's gate / up / down (expert == n_experts: the shared expert)."""
    if naming == NAMING_DSV41:
        p = f"{prefix}.shared_experts" if expert == n_experts else f"{prefix}.experts.{expert}"
        return {"gate": f"{p}.w1", "up": f"{p}.w3", "down": f"{p}.w2"}
    p = f"{prefix}.shared_expert" if expert == n_experts else f"{prefix}.experts.{expert}"
    return {"gate": f"{p}.gate_proj", "up": f"{p}.up_proj", "down": f"{p}.down_proj"}


def moe_checkpoint_tensors(inp, prefix: str, naming: int = NAMING_DSV41,
                           values: Optional[Dict[str, np.ndarray]] = None,
                           value_tag: str = "BF16") -> List[Tuple[str, str, np.ndarray]]:
    """One layer's MoE as (name, dtype tag, array) triples in checkpoint order.  NAMING_DSV41 writes `inp`'s MXFP4 tensors as they are (I8 codes,
    F8_E8M0 scales); NAMING_GLM writes unquantised matrices taken from `values` (name stem -> [out, in] array of
    the numpy type that `value_tag` stands for)."""
    cfg = inp.cfg
    E = cfg.n_experts
    out: List[Tuple[str, str, np.ndarray]] = [(f"{prefix}.gate.weight", "F32", inp.router_w)]
    bias_name = f"{prefix}.gate.bias" if naming == NAMING_DSV41 else f"{prefix}.gate.e_score_correction_bias"
    out.append((bias_name, "F32", inp.router_bias))
    n_src = E + (1 if cfg.shared_inter > 0 else 0)
    for e in range(n_src):
        nm = moe_tensor_names(naming, prefix, e, E)
        if naming == NAMING_DSV41:
            shared = e == E
            for key, wf, sf in (("gate", "gate_w", "gate_s"), ("down", "down_w", "down_s"), ("up", "up_w", "up_s")):
                w = getattr(inp, ("sh_" + wf) if shared else wf)
                s = getattr(inp, ("sh_" + sf) if shared else sf)
                out.append((nm[key] + ".weight", "I8", (w[0] if shared else w[e]).view(np.int8)))
                out.append((nm[key] + ".scale", "F8_E8M0", s[0] if shared else s[e]))
        else:
            for key in ("gate", "down", "up"):
                out.append((nm[key] + ".weight", value_tag, values[nm[key]]))
    return out


def write_moe_checkpoint(path: str, inp, prefix: str, naming: int = NAMING_DSV41,
                         values: Optional[Dict[str, np.ndarray]] = None, value_tag: str = "BF16") -> None:
    """One layer's MoE as a single checkpoint file (see moe_checkpoint_tensors)."""
    write_safetensors(path, moe_checkpoint_tensors(inp, prefix, naming, values, value_tag), metadata={"format": "pt"})
