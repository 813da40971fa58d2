"""Checkpoint -> device on the GPU: a synthetic safetensors shard streamed by the C++ loader into the packed
buffer.  Bars: the packed buffer equals, byte for byte, the one the whole-layer repack builds from the same
tensors; its dequantisation equals the oracle's dequantisation of the file's bytes (quant.rs:260-278); an
unquantised checkpoint (GLM names) equals the oracle's act_quant_fp4 (quant.rs:217-238) of the file's values; the
layer run from the loaded buffer equals the layer run from memory-loaded weights bit for bit."""
import dataclasses

import numpy as np
import pytest
import torch

from ferrite_amd import checkpoint as ck
from ferrite_amd import synth
from ferrite_amd.backend import MODE_MFMA_FP8, InvalidArg

pytestmark = pytest.mark.gpu


def dev(hip, a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(hip.device)


def host(hip, t):
    hip.sync()
    return t.cpu().numpy()


CFG = synth.MoeConfig(name="ck", n=24, hidden=384, n_experts=7, topk=3, inter=384, shared_inter=128, n_group=1,
                      topk_group=1, act_bf16=True)


def _cfg():
    # inter = 384: scale rows of the down matrices hold 12 bytes, not a multiple of 16 (the pitch case)
    assert CFG.inter == 384 and (CFG.inter // 32) % 16 != 0
    return CFG


def _expert_arrays(inp, e):
    E = inp.cfg.n_experts
    if e == E:
        return {k: (getattr(inp, f"sh_{k}_w")[0], getattr(inp, f"sh_{k}_s")[0]) for k in ("gate", "up", "down")}
    return {k: (getattr(inp, f"{k}_w")[e], getattr(inp, f"{k}_s")[e]) for k in ("gate", "up", "down")}


@pytest.mark.parametrize("workers,pad", [(1, False), (3, False), (4, True), (16, True)])
def test_dsv41_shard_loads_into_the_same_packed_bytes(hip, oracle, tmp_path, workers, pad):
    cfg = _cfg()
    inp = synth.make_inputs(cfg, seed=11)
    path = str(tmp_path / "layer.safetensors")
    ck.write_moe_checkpoint(path, inp, "layers.6.ffn", ck.NAMING_DSV41)
    ref_layer = hip.load_moe_layer(inp)
    with ck.Checkpoint(path) as c:
        assert c.validate_moe(cfg, "layers.6.ffn", ck.NAMING_DSV41) == []
        layer, stats = c.load_moe_layer(hip, cfg, "layers.6.ffn", ck.NAMING_DSV41, workers=workers, pad_scale_rows=pad)
    assert stats.workers == min(workers, cfg.n_experts + 1)
    per_expert = 3 * (cfg.hidden * cfg.inter // 2 + cfg.hidden * cfg.inter // 32)
    shared = 3 * (cfg.hidden * cfg.shared_inter // 2 + cfg.hidden * cfg.shared_inter // 32)
    assert stats.source_bytes == cfg.n_experts * per_expert + shared + cfg.n_experts * cfg.hidden * 4 + cfg.n_experts * 4
    assert stats.packed_bytes == layer.packed.numel() == ref_layer.packed.numel()
    assert torch.equal(layer.packed, ref_layer.packed)
    assert np.array_equal(host(hip, layer.tensors["router_bias"]), inp.router_bias)
    for e in (0, cfg.n_experts - 1, cfg.n_experts):
        for which, key in enumerate(("gate", "up", "down")):
            w, s = _expert_arrays(inp, e)[key]
            assert np.array_equal(host(hip, hip.packed_dequant(layer, e, which)), oracle.dequant_fp4_row32(w, s))
    # and the layer runs from it: no checkpoint-layout tensor is on the device
    x = torch.from_numpy(inp.x).to(hip.device).to(torch.bfloat16)
    out_a = torch.empty(cfg.n, cfg.hidden, dtype=torch.float32, device=hip.device)
    out_b = torch.empty_like(out_a)
    hip.moe_layer_dev_mxfp4(layer, x, out_a, MODE_MFMA_FP8)
    hip.moe_layer_dev_mxfp4(ref_layer, x, out_b, MODE_MFMA_FP8)
    hip.sync()
    assert torch.equal(out_a, out_b)


def test_split_checkpoint_loads_like_a_single_file(hip, tmp_path):
    """The layer's tensors dealt over three shard files (as released checkpoints split a layer's experts) load
    into the same packed bytes."""
    cfg = _cfg()
    inp = synth.make_inputs(cfg, seed=15)
    ref_layer = hip.load_moe_layer(inp)
    tensors = ck.moe_checkpoint_tensors(inp, "layers.6.ffn", ck.NAMING_DSV41)
    paths = [str(tmp_path / f"model-{i:05d}-of-00003.safetensors") for i in range(3)]
    for i, p in enumerate(paths):
        ck.write_safetensors(p, tensors[i::3])
    with ck.Checkpoint(paths) as c:
        layer, stats = c.load_moe_layer(hip, cfg, "layers.6.ffn", ck.NAMING_DSV41, workers=5)
    assert torch.equal(layer.packed, ref_layer.packed)
    assert stats.source_bytes == sum(a.nbytes for _, _, a in tensors)
    with ck.Checkpoint(paths[1:]) as c:
        with pytest.raises(InvalidArg, match="missing tensor layers.6.ffn.gate.weight"):
            c.load_moe_layer(hip, cfg, "layers.6.ffn", ck.NAMING_DSV41)


def test_pack_expert_with_padded_scale_rows(hip, oracle):
    """The source pitch argument: scale planes staged with rows padded to 16 bytes (weights.rs:599) and filled with
    junk between the rows give the same packed bytes as dense planes."""
    cfg = _cfg()
    inp = synth.make_inputs(cfg, seed=12)
    ref_layer = hip.load_moe_layer(inp)
    layer = hip.load_moe_layer(inp)
    layer.packed.fill_(0xAB)

    def padded(s, pitch):
        out = np.full((s.shape[0], pitch), 0x5A, np.uint8)
        out[:, :s.shape[1]] = s
        return out

    gu_pitch, dn_pitch = 16, 16                     # hidden/32 = 12 and inter/32 = 12 bytes per row, padded to 16
    for e in range(cfg.n_experts + 1):
        a = _expert_arrays(inp, e)
        inter = cfg.shared_inter if e == cfg.n_experts else cfg.inter
        dpitch = 16 if inter // 32 <= 16 else inter // 32
        pair = lambda k, p: (dev(hip, a[k][0]), dev(hip, padded(a[k][1], p)))
        hip.pack_expert(layer, e, gate=pair("gate", gu_pitch), up=pair("up", gu_pitch), gate_up_scale_pitch=gu_pitch)
        hip.pack_expert(layer, e, down=pair("down", dpitch), down_scale_pitch=dpitch)
    hip.sync()
    import ctypes as C
    rw = dev(hip, inp.router_w)
    assert hip.lib.ferrite_moe_pack_router(C.byref(layer.shape), rw.data_ptr(), layer.packed.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(layer.packed, ref_layer.packed)


def test_pack_expert_error_paths(hip):
    cfg = _cfg()
    inp = synth.make_inputs(cfg, seed=12)
    layer = hip.load_moe_layer(inp)
    a = _expert_arrays(inp, 0)
    g = (dev(hip, a["gate"][0]), dev(hip, a["gate"][1]))
    u = (dev(hip, a["up"][0]), dev(hip, a["up"][1]))
    with pytest.raises(InvalidArg):
        hip.pack_expert(layer, 0)                                  # nothing to pack
    with pytest.raises(InvalidArg):
        hip.pack_expert(layer, 0, gate=g)                          # gate without up
    with pytest.raises(InvalidArg):
        hip.pack_expert(layer, cfg.n_experts + 1, gate=g, up=u)    # expert out of range
    with pytest.raises(InvalidArg):
        hip.pack_expert(layer, -1, gate=g, up=u)
    with pytest.raises(InvalidArg):
        hip.pack_expert(layer, 0, gate=g, up=u, gate_up_scale_pitch=cfg.hidden // 32 - 1)   # pitch below a row
    no_shared = hip.load_moe_layer(synth.make_inputs(dataclasses.replace(cfg, shared_inter=0), seed=12))
    with pytest.raises(InvalidArg):
        hip.pack_expert(no_shared, cfg.n_experts, gate=g, up=u)    # no shared expert in this shape


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mxfp4_quant_bit_exact_vs_oracle(hip, oracle, dtype):
    rng = np.random.default_rng(21)
    x = (rng.normal(0, 1, (48, 256)) * np.repeat(10.0 ** rng.uniform(-6, 6, (48, 8)), 32, axis=1)).astype(np.float32)
    x[1, 0:32] = 0.0                                             # an all-zero block: scale floors at 2^-126
    x[2, 0:32] = -0.0
    # every rounding boundary of the e2m1 grid and its neighbours, at scale 1 (amax 6 -> scale 2^0)
    mids = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], np.float32)
    edge = np.concatenate([mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(9)), [6.0, 0.0, 0.5, 4.0]])
    x[3, 0:25] = edge
    x[3, 25:32] = -mids
    x[4, 0:32] = np.float32(1e-30) * rng.normal(0, 1, 32)        # tiny values: negative ones keep their sign bit
    x[5, 0:32] = np.float32(3e38) * np.sign(rng.normal(0, 1, 32))
    x[6, 0] = 7.0                                                 # amax/6 not a power of two: scale rounds up
    x[7, 0:32] = np.linspace(-6.5, 6.5, 32)
    xt = torch.from_numpy(x).to(dtype)
    xr = xt.to(torch.float32).numpy()
    codes, s = hip.mxfp4_quant(xt.to(hip.device))
    co, so = oracle.act_quant_fp4(xr, 32, True)
    assert np.array_equal(host(hip, codes).ravel(), co)
    sb = host(hip, s).ravel()
    assert sb.min() >= 1 and np.array_equal(np.exp2(sb.astype(np.float64) - 127), so.astype(np.float64))
    # read back through the dequantiser, every value is within half the widest grid spacing (2, from 4 to 6) of
    # its input; the 3e38 block is left out, where 4 * 2^126 is beyond f32
    back = host(hip, hip.mxfp4_dequant(codes, s))
    half_step = np.repeat(so.reshape(48, 8), 32, axis=1).astype(np.float64)
    ok = np.abs(back.astype(np.float64) - xr) <= half_step
    ok[5, 0:32] = True
    assert ok.all()


def _glm_values(cfg, prefix, seed, as_bf16):
    rng = np.random.default_rng(seed)
    values, f32 = {}, {}
    for e in range(cfg.n_experts + 1):
        nm = ck.moe_tensor_names(ck.NAMING_GLM, prefix, e, cfg.n_experts)
        inter = cfg.shared_inter if e == cfg.n_experts else cfg.inter
        for key, shape in (("gate", (inter, cfg.hidden)), ("up", (inter, cfg.hidden)), ("down", (cfg.hidden, inter))):
            v = (rng.normal(0, 0.02, shape) * 2.0 ** rng.integers(-3, 4, (shape[0], 1))).astype(np.float32)
            if as_bf16:
                t = torch.from_numpy(v).to(torch.bfloat16)
                values[nm[key]] = t.view(torch.int16).numpy().view(np.uint16)
                f32[nm[key]] = t.to(torch.float32).numpy()
            else:
                values[nm[key]] = v
                f32[nm[key]] = v
    return values, f32


@pytest.mark.parametrize("as_bf16", [True, False])
def test_glm_shard_is_quantised_on_load(hip, oracle, tmp_path, as_bf16):
    cfg = _cfg()
    prefix = "model.layers.3.mlp"
    inp = synth.make_inputs(cfg, seed=13)
    values, f32 = _glm_values(cfg, prefix, 13, as_bf16)
    path = str(tmp_path / "glm.safetensors")
    ck.write_moe_checkpoint(path, inp, prefix, ck.NAMING_GLM, values=values, value_tag="BF16" if as_bf16 else "F32")
    with ck.Checkpoint(path) as c:
        assert c.validate_moe(cfg, prefix, ck.NAMING_GLM) == []
        layer, stats = c.load_moe_layer(hip, cfg, prefix, ck.NAMING_GLM, workers=3)
    assert np.array_equal(host(hip, layer.tensors["router_bias"]), inp.router_bias)
    for e in (0, 3, cfg.n_experts):
        nm = ck.moe_tensor_names(ck.NAMING_GLM, prefix, e, cfg.n_experts)
        for which, key in enumerate(("gate", "up", "down")):
            v = f32[nm[key]]
            codes, s = oracle.act_quant_fp4(v, 32, True)
            sb = np.round(np.log2(s.astype(np.float64))).astype(np.int64) + 127
            want = oracle.dequant_fp4_row32(codes.reshape(v.shape[0], -1), sb.astype(np.uint8).reshape(v.shape[0], -1))
            assert np.array_equal(host(hip, hip.packed_dequant(layer, e, which)), want), (e, key)
    # the router went in as well: the layer from the loaded buffer routes like one built from the same router
    x = torch.from_numpy(inp.x).to(hip.device).to(torch.bfloat16)
    out = torch.empty(cfg.n, cfg.hidden, dtype=torch.float32, device=hip.device)
    hip.moe_layer_dev_mxfp4(layer, x, out, MODE_MFMA_FP8)
    ids = host(hip, hip.workspace_view(layer, cfg.n, MODE_MFMA_FP8)["ids"])
    ref = oracle.moe_route(oracle.matmul(x.float().cpu().numpy(), inp.router_w), inp.router_bias, cfg.topk,
                           cfg.routed_scaling, cfg.n_group, cfg.topk_group)
    assert np.array_equal(ids, ref[1].astype(np.int32))
    assert torch.isfinite(out).all()


def test_loader_rejects_what_it_cannot_load(hip, tmp_path):
    cfg = _cfg()
    inp = synth.make_inputs(cfg, seed=14)
    good = str(tmp_path / "good.safetensors")
    ck.write_moe_checkpoint(good, inp, "layers.6.ffn", ck.NAMING_DSV41)
    with ck.Checkpoint(good) as c:
        with pytest.raises(InvalidArg, match="missing tensor layers.9.ffn.gate.weight"):
            c.load_moe_layer(hip, cfg, "layers.9.ffn", ck.NAMING_DSV41)
        with pytest.raises(InvalidArg, match=r"experts\.0\.w1\.weight: shape \[384, 192\] != \[512, 192\]"):
            c.load_moe_layer(hip, dataclasses.replace(cfg, inter=512), "layers.6.ffn", ck.NAMING_DSV41)
        with pytest.raises(InvalidArg, match="not supported by the MFMA path"):
            c.load_moe_layer(hip, dataclasses.replace(cfg, hidden=96), "layers.6.ffn", ck.NAMING_DSV41)
        with pytest.raises(InvalidArg, match="missing tensor"):
            c.load_moe_layer(hip, cfg, "layers.6.ffn", ck.NAMING_GLM)

    # rebuild the shard with one tensor changed at a time
    def tensors():
        with ck.Checkpoint(good) as c:
            names = []
            with open(good, "rb") as f:
                import json, struct
                hlen = struct.unpack("<Q", f.read(8))[0]
                hdr = json.loads(f.read(hlen))
                blob = f.read()
            for name, meta in hdr.items():
                if name == "__metadata__":
                    continue
                b, e = meta["data_offsets"]
                names.append([name, meta["dtype"], np.frombuffer(blob[b:e], np.uint8).copy(), meta["shape"]])
            return names

    def rewrite(path, items):
        out = []
        for name, tag, raw, shape in items:
            npdt = {"F32": np.float32, "I8": np.int8, "F8_E8M0": np.uint8, "F8_E4M3": np.uint8, "F16": np.float16}[tag]
            out.append((name, tag, raw.view(npdt).reshape(shape)))
        ck.write_safetensors(path, out)

    bad = str(tmp_path / "bad.safetensors")
    items = tensors()
    for it in items:                                   # the shared expert as the real checkpoint stores it: e4m3
        if ".shared_experts." in it[0] and it[0].endswith(".weight"):
            it[1] = "F8_E4M3"
    rewrite(bad, items)
    with ck.Checkpoint(bad) as c:
        with pytest.raises(InvalidArg, match="shared expert is stored as F8_E4M3"):
            c.load_moe_layer(hip, cfg, "layers.6.ffn", ck.NAMING_DSV41)
        # ... and the routed experts load once the caller takes the shared expert elsewhere
        layer, _ = c.load_moe_layer(hip, dataclasses.replace(cfg, shared_inter=0), "layers.6.ffn", ck.NAMING_DSV41)
        assert layer.packed.numel() > 0
    items = tensors()
    for it in items:
        if it[0] == "layers.6.ffn.experts.2.w3.scale":
            it[1] = "F16"
            it[3] = [it[3][0], it[3][1] // 2]
    rewrite(bad, items)
    with ck.Checkpoint(bad) as c:
        with pytest.raises(InvalidArg, match=r"experts\.2\.w3\.scale: dtype F16"):
            c.load_moe_layer(hip, cfg, "layers.6.ffn", ck.NAMING_DSV41)
    # a shard cut short: the last tensor's range runs past the end of the file
    data = open(good, "rb").read()
    open(bad, "wb").write(data[:-100])
    with ck.Checkpoint(bad) as c:
        with pytest.raises(InvalidArg, match="past the end of the file"):
            c.load_moe_layer(hip, cfg, "layers.6.ffn", ck.NAMING_DSV41)
