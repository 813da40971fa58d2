"""GPU parity of the fused MoE layer against the CPU oracle (and the committed golden vectors).

Bars, all as max|d| / max|ref| of the layer output:
  router ids, probs, logits, permutation tables     bit-exact, every mode
  f32 check mode                                    <= 1e-5  against the f32 oracle (CpuBackend's arithmetic)
  MFMA modes against the oracle evaluated with the same activation quantisation (act_mode 1: e4m3 per 32,
  crates/ferrite-models/src/dsv41/quant.rs:201-214; act_mode 2: two such terms)
                                                    <= 5e-3  (observed: 2e-5 .. 1.2e-3); <= 1e-2 on the 128-row path,
                                                             whose expert outputs pass through bf16 (observed 6e-3)
  two-term MFMA mode against the f32 oracle         <= 2e-2  (the bar for bf16 / fp8 activations; observed ~2e-3)
  one-term MFMA mode against the f32 oracle         <= 8e-2  (three mantissa bits on x and on the SwiGLU output:
                                                             4-5 % by construction; asserted so it cannot grow)"""
import os

import numpy as np
import pytest
import torch

from ferrite_amd import synth
from ferrite_amd.backend import MODE_F32_CHECK, MODE_MFMA_FP8, MODE_MFMA_FP8_X2
from tests.refmath import max_abs_rel

pytestmark = pytest.mark.gpu

TOL_F32 = 1e-5
TOL_MFMA = 5e-3           # against the oracle with the same activation quantisation
TOL_MFMA_BF16_Y = 1e-2    # the same on the 128-row path, which keeps the expert outputs y in bf16 (2^-9 per term)
TOL_X2_VS_F32 = 2e-2      # two-term mode against the f32 oracle
TOL_X1_VS_F32 = 8e-2      # one-term mode against the f32 oracle
ACT_MODE = {MODE_MFMA_FP8: 1, MODE_MFMA_FP8_X2: 2}


def check_mfma(hip, oracle, layer, inp, mode, ref32=None, bf16=False, n_threads=8, check_tables=True):
    """One MFMA-mode run: routing bit-exact, output against the same-quantisation oracle and against the f32 one."""
    out, v = run_layer(hip, layer, inp.x, mode, bf16=bf16)
    if ref32 is None:
        ref32 = oracle.moe_ffn_mxfp4(inp, n_threads=n_threads)
    if check_tables:
        check_routing(v, ref32, oracle, inp.cfg)
    refq = oracle.moe_ffn_mxfp4(inp, act_mode=ACT_MODE[mode], n_threads=n_threads)
    err_q, err_32 = max_abs_rel(out, refq["out"]), max_abs_rel(out, ref32["out"])
    tol_q = TOL_MFMA_BF16_Y if hip.unit_rows(layer, inp.cfg.n, mode) >= 64 else TOL_MFMA
    assert err_q <= tol_q, (mode, err_q)
    assert err_32 <= (TOL_X2_VS_F32 if mode == MODE_MFMA_FP8_X2 else TOL_X1_VS_F32), (mode, err_32)
    return out, v, err_q, err_32


def run_layer(hip, layer, x_np, mode, bf16=False):
    cfg = layer.cfg
    x = torch.from_numpy(x_np).to(hip.device)
    if bf16:
        x = x.to(torch.bfloat16)
    out = torch.empty(x.shape[0], cfg.hidden, dtype=torch.float32, device=hip.device)
    hip.moe_layer_dev_mxfp4(layer, x, out, mode)
    hip.sync()
    v = {k: (t.float() if t.dtype == torch.bfloat16 else t).cpu().numpy()
         for k, t in hip.workspace_view(layer, x.shape[0], mode).items()}
    return out.cpu().numpy(), v


def check_routing(v, ref, oracle, cfg):
    assert np.array_equal(v["logits"], ref["logits"])            # sequential-k chain, bit for bit
    assert np.array_equal(v["ids"], ref["ids"].astype(np.int32))
    assert np.array_equal(v["ids_f32"], ref["ids"])
    assert np.array_equal(v["probs"], ref["probs"])
    t = oracle.moe_permute(v["ids"], cfg.n_experts)
    for k in ("counts", "starts", "perm_map", "gather_src", "active"):
        assert np.array_equal(v[k], t[k]), k
    assert int(v["n_active"][0]) == t["n_active"]


def test_layer_c0_f32_check_mode(hip, oracle):
    inp = synth.make_inputs(synth.CONFIGS["c0"], seed=0)
    layer = hip.load_moe_layer(inp)
    out, v = run_layer(hip, layer, inp.x, MODE_F32_CHECK)
    ref = oracle.moe_ffn_mxfp4(inp)
    check_routing(v, ref, oracle, inp.cfg)
    assert max_abs_rel(out, ref["out"]) <= TOL_F32
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "c0_layer.npz"))
    assert np.array_equal(v["ids"], g["ids"]) and np.array_equal(v["perm_map"], g["perm_map"])
    assert max_abs_rel(out, g["out_f32"]) <= TOL_F32


@pytest.mark.parametrize("mode,key", [(MODE_MFMA_FP8, "out_fp8act"), (MODE_MFMA_FP8_X2, "out_fp8x2")])
def test_layer_c0_mfma_modes(hip, oracle, mode, key):
    inp = synth.make_inputs(synth.CONFIGS["c0"], seed=0)
    layer = hip.load_moe_layer(inp)
    out, v, _, _ = check_mfma(hip, oracle, layer, inp, mode)
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "c0_layer.npz"))
    assert max_abs_rel(out, g[key]) <= TOL_MFMA
    assert hip.unit_rows(layer, inp.cfg.n, mode) == 16


def test_layer_smoke_fixture(hip, oracle):
    """crates/ferrite-kernel/tests/gpu_smoke.rs:437-562 (n=1, H 64 is below the MFMA tile: f32 mode only)."""
    from tests.test_oracle_layer import smoke_fixture
    inp, _ = smoke_fixture()
    layer = hip.load_moe_layer(inp, pack=False)
    out, v = run_layer(hip, layer, inp.x, MODE_F32_CHECK)
    ref = oracle.moe_ffn_mxfp4(inp)
    assert np.array_equal(v["ids"], ref["ids"].astype(np.int32))
    assert np.abs(out - ref["out"]).max() < 1e-4       # the reference test's own tolerance (gpu_smoke.rs:566)


@pytest.mark.parametrize("seed,n", [(1, 1), (2, 3), (3, 17), (4, 40), (12, 90)])
def test_layer_small_shapes_all_modes(hip, oracle, seed, n):
    """Ragged token counts: units of 1..16 rows, more than one unit per expert, experts with no tokens."""
    cfg = synth.MoeConfig(n, 256, 8, 3, 256, 128, 4, 2)
    inp = synth.make_inputs(cfg, seed=seed)
    layer = hip.load_moe_layer(inp)
    ref32 = oracle.moe_ffn_mxfp4(inp)
    out, v = run_layer(hip, layer, inp.x, MODE_F32_CHECK)
    check_routing(v, ref32, oracle, cfg)
    assert max_abs_rel(out, ref32["out"]) <= TOL_F32
    check_mfma(hip, oracle, layer, inp, MODE_MFMA_FP8, ref32)
    check_mfma(hip, oracle, layer, inp, MODE_MFMA_FP8_X2, ref32)


@pytest.mark.parametrize("n,hidden,inter,shared", [(24, 2304, 2304, 2304), (19, 2176, 128, 2432), (5, 4096, 256, 0)])
def test_two_term_long_reductions_stream_their_activations_in_windows(hip, oracle, n, hidden, inter, shared):
    """Two-term activations of a reduction longer than 2048 do not stay in LDS whole: they pass through a ring of
    two 1024-k windows (gate/up when hidden > 2048, down when the intermediate size is).  Lengths that are not
    multiples of the window, units of 1..16 rows, a shared expert whose size differs from the routed ones'."""
    cfg = synth.MoeConfig(n, hidden, 8, 3, inter, shared, 4, 2)
    inp = synth.make_inputs(cfg, seed=n)
    layer = hip.load_moe_layer(inp)
    ref32 = oracle.moe_ffn_mxfp4(inp, n_threads=8)
    check_mfma(hip, oracle, layer, inp, MODE_MFMA_FP8_X2, ref32)
    check_mfma(hip, oracle, layer, inp, MODE_MFMA_FP8, ref32)


def test_declined_mode_falls_back(hip, oracle):
    """A shape the MFMA modes decline (hidden size not a multiple of 128) is declined before anything runs; the host
    mirror then does what the reference's caller does with a declined kernel (cuda.rs:5763-5765): it runs the other
    path, here the f32 mode on the checkpoint-layout weights.  One layer, one call site, a decode-sized and a
    prefill-sized batch; and the two-term mode itself serves both sizes of a shape it accepts."""
    from ferrite_amd.backend import DECLINED, OK
    import ctypes as C
    import dataclasses
    odd = synth.MoeConfig(20, 160, 8, 3, 96, 64, 4, 2)
    inp = synth.make_inputs(odd, seed=1)
    layer = hip.load_moe_layer(inp, pack=False)
    for n in (20, 200):
        # the C ABI itself: declined, no workspace size, nothing enqueued
        assert hip.lib.ferrite_moe_layer_check(C.byref(layer.shape), n, MODE_MFMA_FP8_X2) == DECLINED
        assert hip.lib.ferrite_moe_layer_check(C.byref(layer.shape), n, MODE_MFMA_FP8) == DECLINED
        assert hip.lib.ferrite_moe_layer_check(C.byref(layer.shape), n, MODE_F32_CHECK) == OK
        assert hip.lib.ferrite_moe_layer_workspace_bytes(C.byref(layer.shape), n, MODE_MFMA_FP8_X2) == 0
        assert hip.effective_mode(layer, n, MODE_MFMA_FP8_X2) == MODE_F32_CHECK
        cfg = odd.with_tokens(n)
        x_np = synth.make_activations(cfg, seed=3)
        out, v = run_layer(hip, layer, x_np, MODE_MFMA_FP8_X2)   # the same call for both batch sizes
        ref = oracle.moe_ffn_mxfp4(dataclasses.replace(inp, cfg=cfg, x=x_np), n_threads=8)
        check_routing(v, ref, oracle, cfg)
        assert max_abs_rel(out, ref["out"]) <= TOL_F32
        direct, _ = run_layer(hip, layer, x_np, MODE_F32_CHECK)
        assert np.array_equal(out, direct)                     # the fallen-back call is the f32 call, bit for bit
    # a shape the MFMA modes accept: two-term activations at a decode-sized and at a prefill-sized batch
    small = synth.MoeConfig(20, 256, 8, 3, 256, 128, 4, 2)
    inp = synth.make_inputs(small, seed=1)
    layer = hip.load_moe_layer(inp)
    for n, rows in ((20, 16), (200, 64)):
        cfg = small.with_tokens(n)
        assert hip.lib.ferrite_moe_layer_check(C.byref(layer.shape), n, MODE_MFMA_FP8_X2) == OK
        assert hip.effective_mode(layer, n, MODE_MFMA_FP8_X2) == MODE_MFMA_FP8_X2
        assert hip.unit_rows(layer, n, MODE_MFMA_FP8_X2) == rows
        x_np = synth.make_activations(cfg, seed=3)
        out, v = run_layer(hip, layer, x_np, MODE_MFMA_FP8_X2)
        ref = oracle.moe_ffn_mxfp4(dataclasses.replace(inp, cfg=cfg, x=x_np), act_mode=2, n_threads=8)
        assert np.array_equal(v["ids"], ref["ids"].astype(np.int32))
        assert max_abs_rel(out, ref["out"]) <= (TOL_MFMA_BF16_Y if rows == 64 else TOL_MFMA)


@pytest.fixture
def overrides(hip):
    """Sets library overrides for one test and puts the defaults back afterwards."""
    from ferrite_amd.backend import OVERRIDE_UNIT_ROWS, OVERRIDE_Y_F32
    yield lambda **kw: [hip.set_override({"unit_rows": OVERRIDE_UNIT_ROWS, "y_f32": OVERRIDE_Y_F32}[k], v)
                        for k, v in kw.items()]
    hip.set_override(OVERRIDE_UNIT_ROWS, 0)
    hip.set_override(OVERRIDE_Y_F32, 0)


@pytest.mark.parametrize("seed,n,hidden,inter,shared", [(5, 8, 256, 128, 128), (6, 150, 256, 256, 128),
                                                        (7, 700, 384, 256, 384), (8, 1100, 512, 128, 0)])
def test_unit_rows_128_equals_16(hip, oracle, overrides, seed, n, hidden, inter, shared):
    """The 128-row-unit kernels (both operands tiled through LDS) accumulate over k in the same order as the 16-row
    ones: identical bits when both keep the expert outputs in f32, on ragged units (1..128 rows, several units per
    expert, H/64 not a multiple of the block's 4 items).  By default the 128-row path keeps them in bf16: within the
    MFMA bar of the oracle and within bf16 rounding of the f32 run."""
    cfg = synth.MoeConfig(n, hidden, 8, 3, inter, shared, 4, 2)
    inp = synth.make_inputs(cfg, seed=seed)
    layer = hip.load_moe_layer(inp)
    outs = {}
    for rows in (16, 128):
        overrides(unit_rows=rows, y_f32=1)
        layer._ws.clear()
        outs[rows], v = run_layer(hip, layer, inp.x, MODE_MFMA_FP8)
    assert np.array_equal(outs[16], outs[128])
    overrides(y_f32=0)
    layer._ws.clear()
    out_bf16, v = run_layer(hip, layer, inp.x, MODE_MFMA_FP8)
    assert hip.workspace_view(layer, n, MODE_MFMA_FP8)["y"].dtype == torch.bfloat16
    layer._ws.clear()
    assert max_abs_rel(out_bf16, outs[128]) <= 2.0 ** -7          # (topk + 1) terms, each within 2^-9 of its f32 value
    assert max_abs_rel(out_bf16, oracle.moe_ffn_mxfp4(inp, act_mode=1, n_threads=8)["out"]) <= TOL_MFMA_BF16_Y


@pytest.mark.parametrize("n,hidden,inter,shared,experts", [(700, 4096, 1536, 1536, 8), (300, 1024, 512, 256, 8),
                                                           (520, 7168, 2048, 2048, 8)])
def test_prefill_main_loops_are_bit_identical(hip, overrides, n, hidden, inter, shared, experts):
    """The 128-row units have two main loops: both operands staged through LDS, or the weights streamed into
    registers (blocks of 8 or 4 waves) and only the activations staged.  All accumulate over k in the order of the
    16-row kernels: the same bits at the benchmark's hidden and intermediate sizes (H 4096 / I 1536, H 7168 / I 2048),
    on full and ragged units, with f32 and with bf16 expert outputs."""
    from ferrite_amd.backend import OVERRIDE_PREFILL_TILE
    cfg = synth.MoeConfig(n, hidden, experts, 3, inter, shared, 4 if experts % 4 == 0 else 1, 2 if experts % 4 == 0 else 1)
    inp = synth.make_inputs(cfg, seed=n)
    layer = hip.load_moe_layer(inp, keep_checkpoint_layout=False)
    try:
        for y_f32 in (1, 0):
            outs = {}
            for rows, variant in ((16, 0), (128, 0), (128, 1), (128, 2), (128, 3)):
                if rows == 16 and not y_f32:
                    continue
                overrides(unit_rows=rows, y_f32=y_f32)
                hip.set_override(OVERRIDE_PREFILL_TILE, variant)
                layer._ws.clear()
                outs[(rows, variant)], v = run_layer(hip, layer, inp.x, MODE_MFMA_FP8)
                assert int(v["counts"].max()) > 128   # more than one unit per expert, the last one ragged
            first = next(iter(outs.values()))
            for k, o in outs.items():
                assert np.array_equal(o, first), (y_f32, k)
    finally:
        hip.set_override(OVERRIDE_PREFILL_TILE, 0)
        layer._ws.clear()


@pytest.mark.parametrize("seed,n,hidden,inter,shared", [(6, 150, 256, 256, 128), (7, 700, 384, 256, 384),
                                                        (8, 1100, 512, 128, 0), (9, 520, 4096, 1536, 1536)])
def test_two_term_64_row_units_agree_with_16_row_units(hip, oracle, overrides, seed, n, hidden, inter, shared):
    """Two-term activations on the tiled kernels (64-row units: both planes of a k step against the same weight
    registers) and on the 16-row streaming kernels (a plane after the other per group of four k steps) add the same
    products in a different order: f32 outputs agree to rounding, both sit within the MFMA bar of the two-term oracle
    and inside 2e-2 of the f32 oracle, on ragged units and several units per expert."""
    cfg = synth.MoeConfig(n, hidden, 8, 3, inter, shared, 4, 2)
    inp = synth.make_inputs(cfg, seed=seed)
    layer = hip.load_moe_layer(inp)
    outs = {}
    for rows, want in ((16, 16), (128, 64)):
        overrides(unit_rows=rows, y_f32=1)
        layer._ws.clear()
        assert hip.unit_rows(layer, n, MODE_MFMA_FP8_X2) == want
        outs[want], v = run_layer(hip, layer, inp.x, MODE_MFMA_FP8_X2)
    assert int(v["counts"].max()) > 64
    ref = oracle.moe_ffn_mxfp4(inp, act_mode=2, n_threads=8)
    ref32 = oracle.moe_ffn_mxfp4(inp, n_threads=8)
    assert np.array_equal(v["ids"], ref["ids"].astype(np.int32))
    assert max_abs_rel(outs[64], outs[16]) <= 1e-4
    for o in outs.values():
        assert max_abs_rel(o, ref["out"]) <= TOL_MFMA
        assert max_abs_rel(o, ref32["out"]) <= TOL_X2_VS_F32
    overrides(unit_rows=128, y_f32=0)
    layer._ws.clear()
    out_bf16, _ = run_layer(hip, layer, inp.x, MODE_MFMA_FP8_X2)
    assert max_abs_rel(out_bf16, outs[64]) <= 2.0 ** -7
    assert max_abs_rel(out_bf16, ref["out"]) <= TOL_MFMA_BF16_Y


@pytest.mark.parametrize("variant", [0, 2])
def test_prefill_bf16_expert_rows_are_the_rounded_f32_rows(hip, overrides, variant):
    """The 128-row down kernels hand the expert outputs to the combine step as bf16: packed hardware conversion, then
    an exchange between lanes so that a store instruction writes whole rows.  Every value must be the round-to-
    nearest-even of the f32 value the same kernel writes under the test override (torch's cast states the rounding),
    in full and in ragged units, for the LDS-staged and the weight-streaming kernel."""
    from ferrite_amd.backend import OVERRIDE_PREFILL_TILE
    cfg = synth.MoeConfig(700, 1024, 8, 3, 512, 256, 4, 2)
    inp = synth.make_inputs(cfg, seed=11)
    layer = hip.load_moe_layer(inp, keep_checkpoint_layout=False)
    try:
        hip.set_override(OVERRIDE_PREFILL_TILE, variant)
        ys = {}
        for y_f32 in (1, 0):
            overrides(unit_rows=128, y_f32=y_f32)
            layer._ws.clear()
            _, v = run_layer(hip, layer, inp.x, MODE_MFMA_FP8)
            assert int(v["counts"].max()) > 128 and int(v["counts"].min()) % 16 != 0
            ys[y_f32] = v["y"].copy()   # f32 as written, or the bf16 values widened (exact)
        assert np.isfinite(ys[1]).all() and float(np.abs(ys[1]).max()) > 0
        rounded = torch.from_numpy(ys[1]).to(torch.bfloat16).float().numpy()
        assert not np.array_equal(rounded, ys[1])                       # the f32 run really kept more bits
        assert np.array_equal(rounded.view(np.uint32), ys[0].view(np.uint32))
    finally:
        hip.set_override(OVERRIDE_PREFILL_TILE, 0)
        layer._ws.clear()


def test_layer_c1_decode(hip, oracle):
    """The decode benchmark shape: 32 tokens, H 4096, 128 experts, top-8 of 8 groups, I 1536, bf16 activations.
    The two-term mode is what the benchmark runs: within 2e-2 of the f32 oracle (CpuBackend's arithmetic)."""
    inp = synth.make_inputs(synth.CONFIGS["c1"], seed=0)
    layer = hip.load_moe_layer(inp)
    ref32 = oracle.moe_ffn_mxfp4(inp, n_threads=16)
    out, v = run_layer(hip, layer, inp.x, MODE_F32_CHECK)
    check_routing(v, ref32, oracle, inp.cfg)
    assert max_abs_rel(out, ref32["out"]) <= TOL_F32
    for mode in (MODE_MFMA_FP8_X2, MODE_MFMA_FP8):
        _, _, err_q, err_32 = check_mfma(hip, oracle, layer, inp, mode, ref32, bf16=True, n_threads=16)
        print(f"c1 mode {mode}: vs same-quantisation oracle {err_q:.3e}; vs f32 oracle {err_32:.3e}")


def test_layer_graph_capture_replays(hip, oracle):
    """GraphCapable: capture once, replay with fresh data in the same static buffers; every replay must equal the
    eager result for that input (the launch sequence is routing independent)."""
    cfg = synth.CONFIGS["c0"].with_tokens(24)
    inp = synth.make_inputs(cfg, seed=7)
    layer = hip.load_moe_layer(inp)
    x_static = torch.zeros(24, cfg.hidden, device=hip.device)
    out_static = torch.zeros(24, cfg.hidden, device=hip.device)
    hip.workspace(layer, 24, MODE_MFMA_FP8)          # warm the pool before capture (cuda.rs:627-657)
    hip.moe_layer_dev_mxfp4(layer, x_static, out_static, MODE_MFMA_FP8)
    hip.sync()
    hip.begin_capture()
    hip.moe_layer_dev_mxfp4(layer, x_static, out_static, MODE_MFMA_FP8)
    trace = hip.end_capture()
    assert [r.op for r in trace.ops] == ["moe_layer_mxfp4"]
    for seed in (11, 12, 13, 14):
        x = synth.random_normal(seed, 1, 24 * cfg.hidden).reshape(24, cfg.hidden)
        eager = torch.empty_like(out_static)
        hip.moe_layer_dev_mxfp4(layer, torch.from_numpy(x).to(hip.device), eager, MODE_MFMA_FP8)
        hip.sync()
        x_static.copy_(torch.from_numpy(x))
        torch.cuda.synchronize()
        hip.begin_verify(trace)
        assert hip.end_verify()
        assert torch.equal(out_static, eager)
    hip.graph_destroy(trace)


@pytest.mark.parametrize("mode", [MODE_MFMA_FP8_X2, MODE_MFMA_FP8])
def test_chained_layers_in_one_graph(hip, oracle, mode):
    """The 42-layer decode step in small: four layers with their own weights, each reading the previous one's
    output (out -> x), all on ONE workspace, captured as one graph.  Every replay, on fresh input, equals the eager
    layer-by-layer run bit for bit, and the first layer's routing equals the oracle's: the arrival counters that the
    fused head leaves in the shared workspace, and the tables and activations of the layer before, do not leak from
    one layer into the next."""
    n, n_layers = 48, 4
    cfg = synth.MoeConfig(n, 512, 32, 4, 256, 256, 4, 2)
    inps = [synth.make_inputs(cfg, seed=5, layer=l) for l in range(n_layers)]
    layers = [hip.load_moe_layer(i) for i in inps]
    ws = hip.workspace(layers[0], n, mode)
    x_static = torch.zeros(n, cfg.hidden, device=hip.device)
    bufs = [torch.zeros(n, cfg.hidden, device=hip.device) for _ in range(2)]

    def chain(x_in, outs):
        src = x_in
        for l, ly in enumerate(layers):
            hip.moe_layer_dev_mxfp4(ly, src, outs[l], mode, ws)
            src = outs[l]

    def graph_step():
        src = x_static
        for l, ly in enumerate(layers):
            dst = bufs[l & 1]
            hip.moe_layer_dev_mxfp4(ly, src, dst, mode, ws)
            src = dst

    graph_step()
    hip.sync()
    hip.begin_capture()
    graph_step()
    trace = hip.end_capture()
    assert [r.op for r in trace.ops] == ["moe_layer_mxfp4"] * n_layers
    for seed in (31, 32, 33):
        x = torch.from_numpy(synth.random_normal(seed, 1, n * cfg.hidden).reshape(n, cfg.hidden)).to(hip.device)
        eager = [torch.empty(n, cfg.hidden, device=hip.device) for _ in layers]
        chain(x, eager)
        hip.sync()
        x_static.copy_(x)
        torch.cuda.synchronize()
        hip.begin_verify(trace)
        assert hip.end_verify()
        assert torch.equal(bufs[(n_layers - 1) & 1], eager[-1])
        assert torch.equal(bufs[(n_layers - 2) & 1], eager[-2])
        assert torch.isfinite(eager[-1]).all() and eager[-1].abs().max() > 0
    # the chain's first layer against the oracle (the later layers' inputs are this library's own outputs)
    import dataclasses
    x0 = synth.random_normal(33, 1, n * cfg.hidden).reshape(n, cfg.hidden)
    ref = oracle.moe_ffn_mxfp4(dataclasses.replace(inps[0], x=x0), act_mode=ACT_MODE[mode], n_threads=8)
    assert max_abs_rel(eager[0].cpu().numpy(), ref["out"]) <= TOL_MFMA
    hip.graph_destroy(trace)


def test_decode_step_chain_at_the_benchmark_shape(hip, oracle):
    """Three layers of the 42-layer decode step at its real shape (192 tokens, H 4096, 128 experts, I 1536, two-term
    activations): every layer has its own weights, normalises the previous layer's output and runs on it (the block
    call without hc_post), all on one workspace in one graph.  Every layer's output is compared with the oracle's
    rmsnorm -> layer on the input that layer saw (routing bit-exact), and a replay of the graph on fresh input equals
    the eager chain bit for bit."""
    import dataclasses
    cfg, n_layers = synth.CONFIGS["c4"], 3
    n, mode = cfg.n, MODE_MFMA_FP8_X2
    inps = [synth.make_inputs(cfg, seed=0, layer=l) for l in range(n_layers)]
    layers = [hip.load_moe_layer(i, keep_checkpoint_layout=False) for i in inps]
    g = torch.Generator(device="cpu").manual_seed(2)
    norm_ws = [(torch.rand(cfg.hidden, generator=g) + 0.5) for _ in layers]
    norm_d = [w.to(hip.device) for w in norm_ws]
    bws = hip.block_workspace(layers[0], n, mode)
    assert hip.unit_rows(layers[0], n, mode) == 16
    x_static = torch.zeros(n, cfg.hidden, device=hip.device)

    def chain(src, outs):
        for l, ly in enumerate(layers):
            hip.moe_block_mxfp4(ly, src, norm_d[l], 1e-6, None, None, None, outs[l], mode, workspace=bws)
            src = outs[l]

    x0 = torch.from_numpy(synth.round_to_bf16(inps[0].x)).to(hip.device)
    eager = [torch.empty(n, cfg.hidden, device=hip.device) for _ in layers]
    chain(x0, eager)
    hip.sync()
    src = x0
    for l in range(n_layers):
        x_in = src.cpu().numpy()
        hfn = oracle.rmsnorm(x_in, norm_ws[l].numpy(), 1e-6)
        ref = oracle.moe_ffn_mxfp4(dataclasses.replace(inps[l], x=hfn), act_mode=2, n_threads=16)
        ref32 = oracle.moe_ffn_mxfp4(dataclasses.replace(inps[l], x=hfn), act_mode=0, n_threads=16)
        got = eager[l].cpu().numpy()
        err, err32 = max_abs_rel(got, ref["out"]), max_abs_rel(got, ref32["out"])
        print(f"decode-step chain, layer {l}: vs two-term oracle {err:.3e}, vs f32 oracle {err32:.3e}")
        assert err <= TOL_MFMA and err32 <= TOL_X2_VS_F32
        src = eager[l]
    # the routing tables the last layer left in the shared workspace are the oracle's for the input it saw
    v = {k: t.cpu().numpy() for k, t in hip.workspace_view(layers[-1], n, mode, workspace=bws).items() if k != "y"}
    check_routing(v, ref32, oracle, cfg)
    staged = [torch.empty(n, cfg.hidden, device=hip.device) for _ in layers]
    chain(x_static, staged)
    hip.sync()
    hip.begin_capture()
    chain(x_static, staged)
    trace = hip.end_capture()
    assert [r.op for r in trace.ops] == ["moe_block_mxfp4"] * n_layers
    for seed in (41, 42):
        x = torch.from_numpy(synth.round_to_bf16(synth.random_normal(seed, 1, n * cfg.hidden).reshape(n, cfg.hidden)))
        x = x.to(hip.device)
        chain(x, eager)
        hip.sync()
        x_static.copy_(x)
        torch.cuda.synchronize()
        hip.begin_verify(trace)
        assert hip.end_verify()
        for l in range(n_layers):
            assert torch.equal(staged[l], eager[l])
    hip.graph_destroy(trace)


@pytest.mark.parametrize("n_experts,rows", [(16, 128), (64, 128), (128, 16)])
def test_layer_unfused_head_path(hip, oracle, n_experts, rows):
    """More tokens than the fused routing kernel takes (n > 256): separate router GEMM, routing, three-phase
    permutation and quantisation launches; results must not depend on which head ran.  With 16 and 64 experts the
    average expert sees 16 rows or more (the tiled kernels: 128-row units, 64 with two terms), with 128 it still
    streams the weights (16-row units); both activation formats in each."""
    modes = (MODE_MFMA_FP8, MODE_MFMA_FP8_X2)
    cfg = synth.MoeConfig(300, 256, n_experts, 4, 128, 128, 4, 2)
    inp = synth.make_inputs(cfg, seed=9)
    layer = hip.load_moe_layer(inp)
    assert hip.unit_rows(layer, 300, MODE_MFMA_FP8) == rows
    assert hip.unit_rows(layer, 300, MODE_MFMA_FP8_X2) == min(rows, 64)
    ref32 = oracle.moe_ffn_mxfp4(inp, n_threads=8)
    out, v = run_layer(hip, layer, inp.x, MODE_F32_CHECK)
    check_routing(v, ref32, oracle, cfg)
    assert max_abs_rel(out, ref32["out"]) <= TOL_F32
    for mode in modes:
        check_mfma(hip, oracle, layer, inp, mode, ref32)


@pytest.mark.parametrize("mode", [MODE_MFMA_FP8, MODE_MFMA_FP8_X2])
@pytest.mark.parametrize("n,e,bf16", [(100, 128, False), (200, 128, True), (200, 192, False), (256, 320, True), (65, 64, False)])
def test_layer_fused_head_shapes(hip, oracle, n, e, bf16, mode):
    """The fused routing kernel picks its block shape from n x (blocks of 64 experts): one token per block with a
    wide product ring (up to 256 blocks), one token with a narrow ring so that two blocks share a CU (up to 512),
    two tokens per block beyond that.  Logits, routing and tables are bit-exact in each, for f32 and bf16 input,
    with n odd against the two-token blocks, and above 64 tokens, where the permutation that the last block builds
    spans several 64-token chunks.  Its quantisation blocks write one or two terms."""
    cfg = synth.MoeConfig(n, 384, e, 4, 128, 128, 4, 2, act_bf16=bf16)
    inp = synth.make_inputs(cfg, seed=23)
    layer = hip.load_moe_layer(inp)
    check_mfma(hip, oracle, layer, inp, mode, bf16=bf16)


@pytest.mark.parametrize("n", [40, 700])
def test_layer_all_tokens_on_the_same_experts(hip, oracle, n):
    """Maximum skew: a bias of +50 on three experts of one group makes every token pick exactly those (the sigmoid
    is at most 1), so three experts hold n rows each (full 16- / 128-row units plus a ragged tail) and thirteen hold
    none."""
    cfg = synth.MoeConfig(n, 256, 16, 3, 128, 128, 4, 2)
    inp = synth.make_inputs(cfg, seed=21)
    inp.router_bias[:] = 0.0
    inp.router_bias[[4, 5, 7]] = 50.0
    layer = hip.load_moe_layer(inp)
    ref32 = oracle.moe_ffn_mxfp4(inp, n_threads=8)
    assert set(np.unique(ref32["ids"]).astype(int)) == {4, 5, 7}
    out, v = run_layer(hip, layer, inp.x, MODE_F32_CHECK)
    check_routing(v, ref32, oracle, cfg)
    assert v["counts"].max() == n and (v["counts"] > 0).sum() == 3
    assert max_abs_rel(out, ref32["out"]) <= TOL_F32
    check_mfma(hip, oracle, layer, inp, MODE_MFMA_FP8, ref32)
    if n == 40:      # decode-sized: two full units and a ragged one per expert, two-term
        check_mfma(hip, oracle, layer, inp, MODE_MFMA_FP8_X2, ref32)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("n,experts,hidden", [(300, 128, 256), (1000, 64, 384), (600, 256, 256), (1100, 256, 256),
                                              (2100, 512, 256)])
def test_router_chain_forms(hip, oracle, n, experts, hidden, bf16):
    """Beyond 256 tokens the router chain has three forms, chosen by tokens x expert blocks: four waves that share a
    chunk of the weights through LDS, one token each (300 x 128, 1000 x 64); register-tiled with two tokens per wave
    (600 x 256) or four (1100 x 256; 2100 x 512 with two expert blocks per wave).  All walk the same sequential-k f32
    chain, so logits, ids, probabilities and the permutation tables are the oracle's bit for bit, for f32 and bf16
    activations."""
    cfg = synth.MoeConfig(n, hidden, experts, 4, 128, 128, 8, 4, act_bf16=bf16)
    inp = synth.make_inputs(cfg, seed=n)
    layer = hip.load_moe_layer(inp, keep_checkpoint_layout=False)
    _, v = run_layer(hip, layer, inp.x, MODE_MFMA_FP8, bf16=bf16)
    check_routing(v, oracle.moe_ffn_mxfp4(inp, n_threads=8, want_out=False), oracle, cfg)


def test_layer_error_paths(hip):
    """Argument errors are reported by return code before anything is launched (cuda.rs:411-425 conventions)."""
    from ferrite_amd.backend import Declined, FerriteError, InvalidArg, ShapeMismatch
    cfg = synth.CONFIGS["c0"]
    inp = synth.make_inputs(cfg, seed=0)
    layer = hip.load_moe_layer(inp)
    x = torch.from_numpy(inp.x).to(hip.device)
    out = torch.empty_like(x)
    with pytest.raises(ShapeMismatch):
        hip.moe_layer_dev_mxfp4(layer, x[:, :128].contiguous(), out, MODE_MFMA_FP8)
    with pytest.raises(InvalidArg):
        hip.moe_layer_dev_mxfp4(layer, x, out[:4], MODE_MFMA_FP8)
    with pytest.raises(FerriteError):          # the f32 check mode takes f32 activations only
        hip.moe_layer_dev_mxfp4(layer, x.to(torch.bfloat16), out, MODE_F32_CHECK)
    small = torch.empty(1024, dtype=torch.uint8, device=hip.device)
    with pytest.raises(FerriteError):          # FERRITE_ERR_WORKSPACE
        hip.moe_layer_dev_mxfp4(layer, x, out, MODE_MFMA_FP8, workspace=small)
    # hidden not a multiple of 128: the MFMA mode declines at packing time, the f32 mode still runs
    odd = synth.make_inputs(synth.MoeConfig(4, 64, 8, 2, 64, 64, 1, 1), seed=1)
    with pytest.raises((Declined, InvalidArg)):
        hip.load_moe_layer(odd)
    ly = hip.load_moe_layer(odd, pack=False)
    xo = torch.from_numpy(odd.x).to(hip.device)
    oo = torch.empty_like(xo)
    hip.moe_layer_dev_mxfp4(ly, xo, oo, MODE_F32_CHECK)
    # the library declines the MFMA mode for this shape (return code 2, nothing enqueued); the mirror falls back
    import ctypes as C
    from ferrite_amd.backend import DECLINED
    assert hip.lib.ferrite_moe_layer_check(C.byref(ly.shape), 4, MODE_MFMA_FP8) == DECLINED
    o2 = torch.empty_like(xo)
    hip.moe_layer_dev_mxfp4(ly, xo, o2, MODE_MFMA_FP8)
    hip.sync()
    assert torch.equal(oo, o2)


def _block_case(cfg, seed):
    """Inputs of the FFN half of a decoder layer around a seeded MoE layer: pre-norm stream, norm weight, the nh
    hyper-connection streams and their post/comb mixes (post in (0,2), comb row-stochastic-ish as hc_pre makes them)."""
    import dataclasses
    inp = synth.make_inputs(cfg, seed=seed)
    rng = np.random.default_rng(seed + 100)
    n, H, nh = cfg.n, cfg.hidden, 4
    li = (rng.standard_normal((n, H)) * 3.0).astype(np.float32)
    norm_w = rng.uniform(0.5, 1.5, H).astype(np.float32)
    residual = rng.standard_normal((n, nh, H)).astype(np.float32)
    post = rng.uniform(0.0, 2.0, (n, nh)).astype(np.float32)
    comb = rng.uniform(0.0, 1.0, (n, nh, nh)).astype(np.float32)
    comb /= comb.sum(axis=2, keepdims=True)
    return inp, li, norm_w, residual, post, comb, dataclasses


def _block_oracle(oracle, inp, dc, li, norm_w, eps, residual, post, comb, act_mode):
    hfn = oracle.rmsnorm(li, norm_w, eps)
    ffn = oracle.moe_ffn_mxfp4(dc.replace(inp, x=hfn), act_mode=act_mode, n_threads=8)
    return oracle.hc_post(ffn["out"], residual, post, comb), hfn


@pytest.mark.parametrize("n,hidden,experts", [(8, 256, 16), (40, 256, 16), (150, 256, 16), (200, 384, 192), (300, 512, 64),
                                              (300, 256, 16)])
def test_block_rmsnorm_layer_hc_post(hip, oracle, n, hidden, experts):
    """exec/lib.rs:487-492 as one call: rmsnorm -> MoE FFN -> hc_post.  The normalised activations are bit-exact, so
    routing is; the output keeps the layer's bars (relative to max|ref|).  Up to 256 blocks of the fused routing
    kernel (8, 40, 150 tokens here) rmsnorm runs inside it; beyond that, and with the separate routing launches at
    300 tokens, rmsnorm is a launch of its own.  hc_post runs inside the combine up to 256 tokens, as its own
    launch at 300.  300 tokens on 16 experts is a prefill-sized batch: the tiled kernels (128-row units, 64-row units
    with two-term activations) with bf16 expert outputs."""
    cfg = synth.MoeConfig(n, hidden, experts, 4, 128, 128, 4, 2)
    inp, li, norm_w, residual, post, comb, dc = _block_case(cfg, seed=31)
    layer = hip.load_moe_layer(inp)
    d = lambda a: torch.from_numpy(a).to(hip.device)
    out = torch.empty(n, 4, cfg.hidden, device=hip.device)
    for mode, act_mode, tol in ((MODE_F32_CHECK, 0, TOL_F32), (MODE_MFMA_FP8, 1, TOL_MFMA), (MODE_MFMA_FP8_X2, 2, TOL_MFMA)):
        hip.moe_block_mxfp4(layer, d(li), d(norm_w), 1e-6, d(residual), d(post), d(comb), out, mode)
        hip.sync()
        ref, hfn = _block_oracle(oracle, inp, dc, li, norm_w, 1e-6, residual, post, comb, act_mode)
        if mode != MODE_F32_CHECK and hip.unit_rows(layer, n, mode) >= 64:
            assert n * 4 >= 16 * experts       # an average of 16 rows per expert or more: the tiled kernels
            tol = TOL_MFMA_BF16_Y
        assert max_abs_rel(out.cpu().numpy(), ref) <= tol
        # In the MFMA modes the normalised activations exist only inside the routing kernel (rmsnorm is fused into
        # it); that they are the reference's, bit for bit, shows in the logits it leaves behind
        v = hip.workspace_view(layer, n, mode, workspace=hip.block_workspace(layer, n, mode))
        rr = oracle.moe_ffn_mxfp4(dc.replace(inp, x=hfn), act_mode=0, n_threads=8, want_out=False)
        assert np.array_equal(v["logits"].cpu().numpy(), rr["logits"])
        assert np.array_equal(v["ids"].cpu().numpy(), rr["ids"].astype(np.int32))
        assert np.array_equal(v["probs"].cpu().numpy(), rr["probs"])
    # graph capture of the whole block, replayed on fresh data
    li_s, res_s = d(li).clone(), d(residual).clone()
    nw, po, co = d(norm_w), d(post), d(comb)
    hip.moe_block_mxfp4(layer, li_s, nw, 1e-6, res_s, po, co, out, MODE_MFMA_FP8)
    hip.sync()
    hip.begin_capture()
    hip.moe_block_mxfp4(layer, li_s, nw, 1e-6, res_s, po, co, out, MODE_MFMA_FP8)
    trace = hip.end_capture()
    for seed in (41, 42):
        rng = np.random.default_rng(seed)
        li2 = (rng.standard_normal(li.shape) * 2.0).astype(np.float32)
        res2 = rng.standard_normal(residual.shape).astype(np.float32)
        li_s.copy_(d(li2)); res_s.copy_(d(res2))
        torch.cuda.synchronize()
        hip.begin_verify(trace)
        assert hip.end_verify()
        ref, _ = _block_oracle(oracle, inp, dc, li2, norm_w, 1e-6, res2, post, comb, 1)
        assert max_abs_rel(out.cpu().numpy(), ref) <= TOL_MFMA
    hip.graph_destroy(trace)


@pytest.mark.parametrize("mode", [MODE_MFMA_FP8, MODE_MFMA_FP8_X2])
def test_layer_repeated_calls_same_workspace(hip, oracle, mode):
    """The fused routing kernel keeps arrival counters in the workspace and must leave them cleared."""
    inp = synth.make_inputs(synth.CONFIGS["c0"].with_tokens(40), seed=3)
    layer = hip.load_moe_layer(inp)
    ref = oracle.moe_ffn_mxfp4(inp, act_mode=ACT_MODE[mode])
    first = None
    for _ in range(5):
        out, v = run_layer(hip, layer, inp.x, mode)
        check_routing(v, ref, oracle, inp.cfg)
        first = out if first is None else first
        assert np.array_equal(out, first)
    assert max_abs_rel(first, ref["out"]) <= TOL_MFMA


def test_cpp_host_backend_smoke():
    """The C++ HipBackend (ferrite_amd/host) over the same C ABI: golden.rs values, the gpu_smoke.rs fused-MoE
    fixture against its in-test CPU reference, and capture/replay.  One child process."""
    import subprocess
    from ferrite_amd import build as hip_build
    assert os.path.exists(hip_build.HOST_SMOKE), "build the host side first: python -m ferrite_amd.build"
    res = subprocess.run([hip_build.HOST_SMOKE, hip_build.SO_PATH], capture_output=True, text=True, timeout=120)
    print(res.stdout[-2000:], res.stderr[-2000:])
    assert res.returncode == 0 and "ALL OK" in res.stdout


def _scale_check(hip, oracle, cfg, n_sample, mode, seed=0, unit_tokens=False):
    """Full-size run: routing and permutation bit-exact for every token, layer output against both oracles on a
    token sample, and a size-independent property: the layer is a per-token function, so permuting the tokens
    permutes the output rows bit for bit."""
    inp = synth.make_inputs(cfg, seed=seed)
    layer = hip.load_moe_layer(inp, keep_checkpoint_layout=False)
    out, v = run_layer(hip, layer, inp.x, mode, bf16=cfg.act_bf16)
    ref = oracle.moe_ffn_mxfp4(inp, n_threads=16, want_out=False)
    check_routing(v, ref, oracle, cfg)
    sel = np.linspace(0, cfg.n - 1, n_sample).astype(np.int32)
    sub = oracle.moe_ffn_mxfp4(inp, act_mode=ACT_MODE[mode], n_threads=16, tok_sel=sel)
    sub32 = oracle.moe_ffn_mxfp4(inp, act_mode=0, n_threads=16, tok_sel=sel)
    err, err32 = max_abs_rel(out[sel], sub["out"]), max_abs_rel(out[sel], sub32["out"])
    counts = v["counts"]
    print(f"{cfg.name}: sample err {err:.3e} (vs f32 oracle {err32:.3e}); tokens/expert max {counts.max()} "
          f"mean {counts.mean():.1f}; experts hit {(counts > 0).sum()}")
    assert err <= (TOL_MFMA_BF16_Y if hip.unit_rows(layer, cfg.n, mode) >= 64 else TOL_MFMA)
    assert err32 <= (TOL_X2_VS_F32 if mode == MODE_MFMA_FP8_X2 else TOL_X1_VS_F32)
    if unit_tokens:
        # Every row of the first and of the last unit of one expert at this shape (evenly spaced tokens touch a
        # unit's first rows at best).  The tiled kernels cut an expert's rows into ceil(rows / cap) units balanced in
        # whole 16-row tiles (the first units hold one tile more): take the expert with several units whose last
        # unit ends in the emptiest ragged tile.
        rows = hip.unit_rows(layer, cfg.n, mode)
        cand = [e for e in range(cfg.n_experts) if counts[e] > rows and counts[e] % 16]
        e = min(cand, key=lambda i: counts[i] % 16)
        start, cnt = int(v["starts"][e]), int(counts[e])
        units, tiles = -(-cnt // rows), -(-cnt // 16)
        base, rem = divmod(tiles, units)
        first_rows = (base + (1 if rem else 0)) * 16
        last0 = ((units - 1) * base + min(units - 1, rem)) * 16
        assert first_rows <= rows and 0 < cnt - last0 <= rows
        grouped = np.concatenate([np.arange(start, start + first_rows), np.arange(start + last0, start + cnt)])
        toks = np.unique(v["gather_src"][grouped] // cfg.topk).astype(np.int32)
        assert len(toks) == len(grouped)   # an expert holds a token once
        u = oracle.moe_ffn_mxfp4(inp, act_mode=ACT_MODE[mode], n_threads=16, tok_sel=toks)
        err_u = max_abs_rel(out[toks], u["out"])
        print(f"{cfg.name}: expert {e} ({cnt} rows in {units} units): all {first_rows} rows of its first unit and the "
              f"{cnt - last0} rows of its last one, {len(toks)} tokens: err {err_u:.3e}")
        assert err_u <= (TOL_MFMA_BF16_Y if rows >= 64 else TOL_MFMA)
    perm = np.random.default_rng(1).permutation(cfg.n)
    out_p, _ = run_layer(hip, layer, inp.x[perm], mode, bf16=cfg.act_bf16)
    assert np.array_equal(out_p, out[perm])
    return v


@pytest.mark.parametrize("mode", [MODE_MFMA_FP8, MODE_MFMA_FP8_X2])
def test_layer_c2_prefill_scale(hip, oracle, mode):
    """4096 tokens, ~256 tokens per expert: one-term activations on 128-row units (the reference's serving format,
    within 8e-2 of the f32 oracle) and two-term activations on 64-row units (within 2e-2 of it)."""
    _scale_check(hip, oracle, synth.CONFIGS["c2"], n_sample=12, mode=mode, unit_tokens=True)


@pytest.mark.parametrize("mode", [MODE_MFMA_FP8_X2, MODE_MFMA_FP8])
def test_layer_c4_decode192(hip, oracle, mode):
    """One layer of the 42-layer decode step: 192 tokens, about twelve rows per expert."""
    _scale_check(hip, oracle, synth.CONFIGS["c4"], n_sample=12, mode=mode)


def test_layer_c3_skewed_scale(hip, oracle):
    """DeepSeek-V3-scale layer with a Zipf(1.1) correction bias: about 10 % of the experts take about half of the
    assignments; stresses the three-phase permutation and experts with thousands of rows."""
    cfg = synth.CONFIGS["c3"]
    v = _scale_check(hip, oracle, cfg, n_sample=6, mode=MODE_MFMA_FP8, unit_tokens=True)
    counts = np.sort(v["counts"])[::-1]
    top = counts[: cfg.n_experts // 10].sum() / counts.sum()
    assert 0.35 <= top <= 0.65, top
