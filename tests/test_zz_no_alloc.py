"""ferrite_moe_layer_mxfp4_static: the layer on the library's built-in workspace (no allocation anywhere).

Its output must equal ferrite_moe_layer_mxfp4's bit for bit: on two calls in a row, the second with fewer tokens
(the array still holds the first call's tables, counters and activations), in both arithmetic modes, for the fused
head and for the separate routing launches; under a captured graph; and a call too large for the array is refused
with both sizes in the message."""
import ctypes as C

import numpy as np
import pytest
import torch

from ferrite_amd import synth
from ferrite_amd.backend import (MODE_F32_CHECK, MODE_MFMA_FP8, MODE_MFMA_FP8_X2, STATIC_WORKSPACE_BYTES,
                                 FerriteError)

pytestmark = pytest.mark.gpu


def both(hip, layer, x_np, mode, bf16=False):
    x = torch.from_numpy(x_np).to(hip.device)
    if bf16:
        x = x.to(torch.bfloat16)
    want = torch.empty(x.shape[0], layer.cfg.hidden, dtype=torch.float32, device=hip.device)
    got = torch.full_like(want, float("nan"))
    hip.moe_layer_dev_mxfp4(layer, x, want, mode)
    hip.moe_layer_dev_mxfp4_static(layer, x, got, mode)
    hip.sync()
    return got.cpu().numpy(), want.cpu().numpy()


@pytest.mark.parametrize("mode", [MODE_MFMA_FP8, MODE_MFMA_FP8_X2, MODE_F32_CHECK])
def test_static_workspace_equals_caller_workspace_twice_second_smaller(hip, mode):
    cfg = synth.MoeConfig(40, 256, 8, 3, 256, 128, 4, 2)
    inp = synth.make_inputs(cfg, seed=3)
    layer = hip.load_moe_layer(inp)
    got, want = both(hip, layer, inp.x, mode)
    assert np.isfinite(want).all() and np.array_equal(got, want)
    small = synth.make_inputs(cfg.with_tokens(17), seed=4)
    got, want = both(hip, layer, small.x, mode)
    assert np.isfinite(want).all() and np.array_equal(got, want)
    # and back up again: nothing of the smaller call's state may leak into a larger one
    got, want = both(hip, layer, inp.x, mode)
    assert np.array_equal(got, want)


def test_static_workspace_separate_routing_launches_and_bf16(hip):
    """More than 256 tokens: router GEMM, routing, three-phase permutation (its masks live in the workspace) and
    quantisation as separate launches; then a smaller bf16 call through the fused head."""
    cfg = synth.MoeConfig(700, 256, 16, 4, 128, 128, 4, 2)
    inp = synth.make_inputs(cfg, seed=5)
    layer = hip.load_moe_layer(inp)
    got, want = both(hip, layer, inp.x, MODE_MFMA_FP8)
    assert np.isfinite(want).all() and np.array_equal(got, want)
    small = synth.make_inputs(cfg.with_tokens(33), seed=6)
    got, want = both(hip, layer, small.x, MODE_MFMA_FP8, bf16=True)
    assert np.isfinite(want).all() and np.array_equal(got, want)


def test_static_workspace_decode_shape(hip):
    """The decode benchmark shape (32 tokens, H 4096, 128 experts, top-8, I 1536) fits the built-in workspace."""
    inp = synth.make_inputs(synth.CONFIGS["c1"], seed=0)
    layer = hip.load_moe_layer(inp, keep_checkpoint_layout=False)
    for mode in (MODE_MFMA_FP8_X2, MODE_MFMA_FP8):
        got, want = both(hip, layer, inp.x, mode, bf16=True)
        assert np.isfinite(want).all() and np.array_equal(got, want)
        got, want = both(hip, layer, inp.x[:5], mode, bf16=True)
        assert np.array_equal(got, want)


def test_static_workspace_under_graph_capture(hip):
    """Captured once (the counter-clearing launch is a kernel, not a memset node), replayed on fresh inputs with
    eager work in between; every replay equals the eager result."""
    cfg = synth.CONFIGS["c0"].with_tokens(24)
    inp = synth.make_inputs(cfg, seed=7)
    layer = hip.load_moe_layer(inp)
    xs = torch.zeros(24, cfg.hidden, device=hip.device)
    outs = torch.zeros(24, cfg.hidden, device=hip.device)
    hip.moe_layer_dev_mxfp4_static(layer, xs, outs, MODE_MFMA_FP8)
    hip.sync()
    hip.begin_capture()
    hip.moe_layer_dev_mxfp4_static(layer, xs, outs, MODE_MFMA_FP8)
    trace = hip.end_capture()
    for seed in (21, 22, 23):
        x = torch.from_numpy(synth.random_normal(seed, 1, 24 * cfg.hidden).reshape(24, cfg.hidden)).to(hip.device)
        eager = torch.empty_like(outs)
        hip.moe_layer_dev_mxfp4(layer, x, eager, MODE_MFMA_FP8)
        hip.sync()
        xs.copy_(x)
        torch.cuda.synchronize()
        hip.begin_verify(trace)
        assert hip.end_verify()
        assert torch.equal(outs, eager)
    hip.graph_destroy(trace)


def test_static_workspace_refuses_what_does_not_fit(hip):
    cfg = synth.MoeConfig(4000, 256, 16, 4, 128, 128, 4, 2)
    inp = synth.make_inputs(cfg, seed=8)
    layer = hip.load_moe_layer(inp)
    need = hip.lib.ferrite_moe_layer_workspace_bytes(C.byref(layer.shape), cfg.n, MODE_MFMA_FP8)
    assert need > STATIC_WORKSPACE_BYTES
    x = torch.from_numpy(inp.x).to(hip.device)
    out = torch.empty_like(x)
    with pytest.raises(FerriteError, match=f"needs {need} bytes.*holds {STATIC_WORKSPACE_BYTES}"):
        hip.moe_layer_dev_mxfp4_static(layer, x, out, MODE_MFMA_FP8)
