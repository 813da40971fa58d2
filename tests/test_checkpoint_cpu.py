"""Checkpoint reader (C++ host library) on the CPU: the safetensors header index against an independent
implementation (the `safetensors` package), the error wording of the reference's reader
(crates/ferrite-models/src/dsv41/weights.rs:833-880), and the tensor names / on-disk shapes of one layer's MoE
(weights.rs:333-354, the headline names of its own test :908-955; GLM names crates/ferrite-model/src/weights.rs:133-149).
No device work happens here: opening a shard only parses and maps it."""
import json
import os
import re
import struct

import numpy as np
import pytest

from ferrite_amd import checkpoint as ck
from ferrite_amd import synth
from ferrite_amd.backend import InvalidArg

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_host_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "ferrite_amd", "host", "ferrite_host.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = sorted(set(re.findall(r"\b(ferrite_ckpt_[a-z0-9_]+)\s*\(", hdr)))
    lib = ck.load_host_library()
    for name in declared:
        assert hasattr(lib, name), name
    assert declared == sorted(ck.HOST_EXPORTS)


def _raw(path, view, data_start):
    with open(path, "rb") as f:
        f.seek(data_start + view.begin)
        return f.read(view.end - view.begin)


def test_reader_agrees_with_the_safetensors_package(tmp_path):
    from safetensors.numpy import save_file
    rng = np.random.default_rng(0)
    tensors = {
        "layers.0.ffn.gate.weight": rng.standard_normal((16, 256)).astype(np.float32),
        "layers.0.ffn.experts.0.w1.weight": rng.integers(-128, 128, (128, 128), dtype=np.int8),
        "a.scalar": np.array(3.5, np.float32),
        "z.bytes é \"quoted\"": rng.integers(0, 256, (3, 5, 7), dtype=np.uint8),
        "empty": np.zeros((0, 4), np.float32),
        "i64": np.arange(6, dtype=np.int64).reshape(2, 3),
    }
    path = str(tmp_path / "lib.safetensors")
    save_file(tensors, path, metadata={"format": "pt", "note": "x"})
    with ck.Checkpoint(path) as c:
        assert len(c) == len(tensors)          # __metadata__ is not a tensor
        assert c.tensor("__metadata__") is None
        assert c.tensor("absent") is None
        want_tag = {np.dtype(np.float32): "F32", np.dtype(np.int8): "I8", np.dtype(np.uint8): "U8",
                    np.dtype(np.int64): "I64"}
        for name, arr in tensors.items():
            v = c.tensor(name)
            assert v is not None, name
            assert v.dtype == want_tag[arr.dtype]
            assert v.shape == tuple(arr.shape)
            assert _raw(path, v, c.data_start) == arr.tobytes()


def test_writer_is_read_back_by_the_safetensors_package_and_by_the_reader(tmp_path):
    from safetensors import safe_open
    rng = np.random.default_rng(1)
    items = [("b.second", "F32", rng.standard_normal((4, 8)).astype(np.float32)),
             ("a.first", "I8", rng.integers(-128, 128, (2, 16), dtype=np.int8)),
             ("c.scale", "U8", rng.integers(0, 256, (2, 1), dtype=np.uint8))]
    path = str(tmp_path / "mine.safetensors")
    ck.write_safetensors(path, items, metadata={"format": "pt"})
    with safe_open(path, framework="np") as f:
        assert sorted(f.keys()) == sorted(n for n, _, _ in items)
        for name, _, arr in items:
            assert np.array_equal(f.get_tensor(name), arr)
    with ck.Checkpoint(path) as c:
        off = 0
        for name, tag, arr in items:                      # written back to back in the given order
            v = c.tensor(name)
            assert (v.dtype, v.shape, v.begin, v.end) == (tag, arr.shape, off, off + arr.nbytes)
            off += arr.nbytes
        assert c.data_start % 8 == 0


def test_e8m0_tag_is_kept(tmp_path):
    path = str(tmp_path / "e8m0.safetensors")
    ck.write_safetensors(path, [("x.scale", "F8_E8M0", np.full((4, 2), 120, np.uint8))])
    with ck.Checkpoint(path) as c:
        assert c.tensor("x.scale").dtype == "F8_E8M0"


def _write_raw(path, header_bytes, hlen=None, payload=b""):
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(header_bytes) if hlen is None else hlen))
        f.write(header_bytes)
        f.write(payload)


def test_reader_errors_follow_the_reference(tmp_path):  # weights.rs:833-852
    with pytest.raises(InvalidArg, match=r"^open .*missing\.safetensors: "):
        ck.Checkpoint(str(tmp_path / "missing.safetensors"))
    p = str(tmp_path / "short.safetensors")
    open(p, "wb").write(b"\x01\x02\x03")
    with pytest.raises(InvalidArg, match="header len"):
        ck.Checkpoint(p)
    _write_raw(p, b"{}", hlen=100 * 1024 * 1024 + 1)
    with pytest.raises(InvalidArg, match="implausible header length 104857601"):
        ck.Checkpoint(p)
    _write_raw(p, b"{}", hlen=64)
    with pytest.raises(InvalidArg, match="header body"):
        ck.Checkpoint(p)
    for bad in (b'{"a": ', b'{"a" 1}', b'{"a": [1, 2}', b'{"a": "\\q"}', b'{"a": 1} x', b'{a: 1}', b''):
        _write_raw(p, bad)
        with pytest.raises(InvalidArg, match="header json"):
            ck.Checkpoint(p)
    _write_raw(p, b"[1, 2, 3]")
    with pytest.raises(InvalidArg, match="safetensors header is not an object"):
        ck.Checkpoint(p)


def test_reader_handles_json_the_format_allows(tmp_path):
    hdr = {"__metadata__": {"k": "v"}, "tür \U0001F600": {"dtype": "F32", "shape": [2, 3], "data_offsets": [0, 24]},
           "lenient": {"shape": [1]}}
    js = json.dumps(hdr, ensure_ascii=True).encode()     # \\u escapes, a surrogate pair among them
    p = str(tmp_path / "j.safetensors")
    _write_raw(p, js + b"   \n", payload=b"\0" * 24)
    with ck.Checkpoint(p) as c:
        assert len(c) == 2
        v = c.tensor("tür \U0001F600")
        assert (v.dtype, v.shape, v.begin, v.end) == ("F32", (2, 3), 0, 24)
        v = c.tensor("lenient")                           # missing fields read as empty, as in the reference
        assert (v.dtype, v.shape, v.begin, v.end) == ("", (1,), 0, 0)


def _tiny_cfg():
    return synth.MoeConfig(name="t", n=4, hidden=256, n_experts=4, topk=2, inter=128, shared_inter=128, n_group=1,
                           topk_group=1)


def test_moe_names_and_shapes_dsv41(tmp_path):
    cfg = _tiny_cfg()
    inp = synth.make_inputs(cfg, seed=0)
    p = str(tmp_path / "l6.safetensors")
    ck.write_moe_checkpoint(p, inp, "layers.6.ffn", ck.NAMING_DSV41)
    with ck.Checkpoint(p) as c:
        # names the reference's own test lists (weights.rs:908-955), at this layer
        for name in ("layers.6.ffn.gate.weight", "layers.6.ffn.gate.bias", "layers.6.ffn.experts.0.w1.weight",
                     "layers.6.ffn.experts.0.w1.scale", "layers.6.ffn.experts.3.w3.scale",
                     "layers.6.ffn.shared_experts.w2.weight"):
            assert c.tensor(name) is not None, name
        v = c.tensor("layers.6.ffn.experts.2.w2.weight")   # down: [dim, inter/2], one byte per two values
        assert (v.dtype, v.shape) == ("I8", (cfg.hidden, cfg.inter // 2))
        v = c.tensor("layers.6.ffn.experts.2.w2.scale")    # one e8m0 byte per (row, 32 columns)
        assert (v.dtype, v.shape) == ("F8_E8M0", (cfg.hidden, cfg.inter // 32))
        assert len(c) == 2 + 6 * (cfg.n_experts + 1)
        assert c.validate_moe(cfg, "layers.6.ffn", ck.NAMING_DSV41) == []
        missing = c.validate_moe(cfg, "layers.7.ffn", ck.NAMING_DSV41)
        assert len(missing) == len(c) and "layers.7.ffn.gate.weight" in missing
        import dataclasses
        wrong = dataclasses.replace(cfg, inter=256)
        report = c.validate_moe(wrong, "layers.6.ffn", ck.NAMING_DSV41)
        assert "layers.6.ffn.experts.0.w1.weight: shape [128, 128] != [256, 128]" in report
        assert "layers.6.ffn.gate.weight" not in " ".join(report)
        more = dataclasses.replace(cfg, n_experts=5)
        report = c.validate_moe(more, "layers.6.ffn", ck.NAMING_DSV41)
        assert "layers.6.ffn.experts.4.w1.weight" in report
        # a GLM reader finds none of the expert tensors under these names
        assert "layers.6.ffn.experts.0.gate_proj.weight" in c.validate_moe(cfg, "layers.6.ffn", ck.NAMING_GLM)


def test_moe_names_glm(tmp_path):
    cfg = _tiny_cfg()
    inp = synth.make_inputs(cfg, seed=0)
    rng = np.random.default_rng(0)
    values = {}
    for e in range(cfg.n_experts + 1):
        nm = ck.moe_tensor_names(ck.NAMING_GLM, "model.layers.3.mlp", e, cfg.n_experts)
        inter = cfg.shared_inter if e == cfg.n_experts else cfg.inter
        values[nm["gate"]] = rng.integers(0, 65536, (inter, cfg.hidden), dtype=np.uint16)
        values[nm["up"]] = rng.integers(0, 65536, (inter, cfg.hidden), dtype=np.uint16)
        values[nm["down"]] = rng.integers(0, 65536, (cfg.hidden, inter), dtype=np.uint16)
    p = str(tmp_path / "glm.safetensors")
    ck.write_moe_checkpoint(p, inp, "model.layers.3.mlp", ck.NAMING_GLM, values=values)
    with ck.Checkpoint(p) as c:
        for name in ("model.layers.3.mlp.gate.weight", "model.layers.3.mlp.gate.e_score_correction_bias",
                     "model.layers.3.mlp.shared_expert.gate_proj.weight", "model.layers.3.mlp.experts.3.down_proj.weight"):
            assert c.tensor(name) is not None, name
        assert c.tensor("model.layers.3.mlp.experts.1.up_proj.weight").shape == (cfg.inter, cfg.hidden)
        assert c.validate_moe(cfg, "model.layers.3.mlp", ck.NAMING_GLM) == []


def test_split_checkpoint_takes_each_tensor_from_the_shard_that_names_it(tmp_path):
    cfg = _tiny_cfg()
    inp = synth.make_inputs(cfg, seed=0)
    tensors = ck.moe_checkpoint_tensors(inp, "layers.6.ffn", ck.NAMING_DSV41)
    paths = [str(tmp_path / f"model-{i:05d}-of-00003.safetensors") for i in range(3)]
    for i, p in enumerate(paths):                       # tensors dealt round-robin over three files
        ck.write_safetensors(p, tensors[i::3], metadata={"format": "pt"})
    with ck.Checkpoint(paths) as c:
        assert len(c) == len(tensors)
        assert c.validate_moe(cfg, "layers.6.ffn", ck.NAMING_DSV41) == []
        for name, tag, arr in tensors:
            v = c.tensor(name)
            assert (v.dtype, v.shape) == (tag, arr.shape), name
    with ck.Checkpoint(paths[:2]) as c:                  # a shard short: its tensors are reported by name
        missing = c.validate_moe(cfg, "layers.6.ffn", ck.NAMING_DSV41)
        assert sorted(missing) == sorted(n for n, _, _ in tensors[2::3])
    with pytest.raises(InvalidArg, match=r"^open .*absent\.safetensors: "):
        ck.Checkpoint([paths[0], str(tmp_path / "absent.safetensors")])
    with pytest.raises(InvalidArg):
        ck.Checkpoint([])
