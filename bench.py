#!/usr/bin/env python3
"""Benchmark of the MoE FFN layer on one MI355X.

One "step" = one pass of the fused layer (router GEMM -> routing -> permutation -> activation quantisation ->
gate/up GEMM + SwiGLU -> down GEMM -> combine) over one batch of synthetic tokens, replayed from a captured
hipGraph the way a decode step runs in production.  Inputs and weights are resident in HBM before the timed
region.  Prints ONE JSON line: metric / value (tokens per second of the layer) / ms_per_step and the workload in
"config"; "roofline" for the gate/up kernel (algorithmic bytes or flops per launch over its duration, measured with
HIP events on the launch stream; "traffic" = counter-derived HBM bytes per launch of the profiled build);
"cpu_baseline" (the CPU oracle on the same tokens); and the legs described below.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c1] [--no-cpu-baseline]

The default run times the decode layer (c1: 32 tokens, two-term activations; "decode_fp8": the same with one term)
and, on the same weights, a bounded prefill leg (c2: 4096 tokens, one-term activations, with its own roofline and
distance to the f32 oracle, and "two_term": the same chunk with two-term activations) reported under "prefill";
"decode_step" is the 42-layer decode step (c4: 192 tokens): every layer has its own weights, the layers are chained
(rmsnorm of a layer's output is the next layer's input) and share one workspace, and the whole step is one
hipGraph (--config c4 times that step alone).  "block_rmsnorm_layer_hc_post" and "checkpoint_load" time the steps
either side of the layer.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
MFMA_PEAK_FP8_TFLOPS = 5000.0  # dense fp8-operand MFMA (e4m3 activations x e2m1 weights run at this rate)
MFMA_PEAK_FP4_TFLOPS = 10100.0 # dense MXFP4 x MXFP4

# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by the same
# counters' reading for a 1 GiB device copy (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000); the runs and raw values
# are in profiles/.  Counters cannot be read inside this script, so each figure carries the build id of the
# library it was measured on: a run on another build reports traffic null and names the profiled build.
MEASURED_TRAFFIC = {}   # (config, kernel) -> (bytes per launch, build id); filled in from profiles/ below
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "measured_traffic.json")
if os.path.exists(TRAFFIC_FILE):
    with open(TRAFFIC_FILE) as _f:
        for _e in json.load(_f)["entries"]:
            MEASURED_TRAFFIC[(_e["config"], _e["kernel"])] = (_e["bytes_per_launch"], _e["build_id"])

WORKLOADS = {
    "c0": "c0: tiny parity layer, 8 tokens, H256 E16 top4 (4 groups/2) I128, MXFP4 weights, f32 activations",
    "c1": "c1: GLM-5.3-Flash-shaped decode MoE layer, 32 tokens, H4096 E128+1 shared top8 (8 groups/4) I1536, "
          "MXFP4 weights, bf16 activations",
    "c2": "c2: same layer at prefill chunk, 4096 tokens, e4m3/32 activations",
    "c3": "c3: DeepSeek-V3-scale skewed layer, 8192 tokens, H7168 E256+1 top8 (8 groups/4) I2048, Zipf(1.1) bias",
    "c4": "c4: 42-MoE-layer decode step of the GLM-5.3-Flash shape at 192 tokens (batch 64 x MTP 3), all layers in one "
          "hipGraph; every layer has its own weights (54 GB resident); the layers are chained, each reading the "
          "rmsnorm of the previous layer's output, and share one workspace",
}


class HipEvents:
    """hipEvent_t handles through the HIP runtime (events must live on the stream the kernels run on)."""

    def __init__(self):
        self.rt = C.CDLL("libamdhip64.so")
        self.rt.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.rt.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.rt.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.rt.hipEventSynchronize.argtypes = [C.c_void_p]
        self.rt.hipEventDestroy.argtypes = [C.c_void_p]

    def create(self, n):
        evs = (C.c_void_p * n)()
        for i in range(n):
            e = C.c_void_p()
            if self.rt.hipEventCreate(C.byref(e)) != 0:
                raise RuntimeError("hipEventCreate failed")
            evs[i] = e
        return evs

    def elapsed_ms(self, a, b) -> float:
        ms = C.c_float()
        rc = self.rt.hipEventElapsedTime(C.byref(ms), a, b)
        if rc != 0:
            raise RuntimeError(f"hipEventElapsedTime rc={rc}")
        return ms.value

    def destroy(self, evs):
        for e in evs:
            self.rt.hipEventDestroy(e)


def algorithmic_bytes(cfg, n, n_active):
    """HBM bytes the layer has to move once (weights of the experts that are hit + shared, router, x, out)."""
    H, I, Is, E = cfg.hidden, cfg.inter, cfg.shared_inter, cfg.n_experts
    per_mat = lambda rows, cols: rows * cols // 2 + rows * cols // 32
    gate_up = n_active * 2 * per_mat(I, H) + (2 * per_mat(Is, H) if Is else 0)
    down = n_active * per_mat(H, I) + (per_mat(H, Is) if Is else 0)
    router = E * H * 4
    act = n * H * 2 * 2
    return dict(gate_up=gate_up, down=down, router=router, act=act, total=gate_up + down + router + act)


def time_replays(hip, torch, launch, steps, warmup):
    """Seconds per call of `launch` over exactly `steps` calls, synchronised on both sides."""
    for _ in range(warmup):
        launch()
    hip.sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        launch()
    hip.sync()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def stage_profile(hip, ev, layer, x, out, mode, ws, reps):
    """Per-stage durations from eager launches with HIP events recorded on the launch stream between the stages,
    plus the gate/up kernel itself (events that bracket its execution on the device: what rocprofv3 reports)."""
    sets = [ev.create(10) for _ in range(reps)]
    for s in sets:
        hip.moe_layer_dev_mxfp4(layer, x, out, mode, ws, stage_events=s)
    hip.sync()
    names = ["router_gemm", "route", "permute", "act_quant", "gate_up_mfma", "down_mfma", "combine"]
    stage_us = {nm: float(np.mean([ev.elapsed_ms(s[i], s[i + 1]) for s in sets]) * 1e3) for i, nm in enumerate(names)}
    eager_us = float(np.mean([ev.elapsed_ms(s[0], s[7]) for s in sets]) * 1e3)
    gu_kernel_us = float(np.mean([ev.elapsed_ms(s[8], s[9]) for s in sets]) * 1e3)
    for s in sets:
        ev.destroy(s)
    return stage_us, eager_us, gu_kernel_us


def measured_traffic(config, kernel, build_id):
    """{"traffic": bytes or None[, "traffic_stale_build": id]} for the roofline object."""
    hit = MEASURED_TRAFFIC.get((config, kernel))
    if hit is None:
        return {"traffic": None}
    if hit[1] != build_id:
        return {"traffic": None, "traffic_stale_build": hit[1], "traffic_of_that_build": hit[0]}
    return {"traffic": hit[0]}


def gate_up_roofline(cfg, n, unit_rows, gu_us, ab, config_name, build_id):
    if unit_rows < 64:
        # decode-sized batch: every weight byte is streamed once per unit; the kernel is HBM bound
        gbs = ab["gate_up"] / (gu_us * 1e-6) / 1e9
        r = {"bound": "hbm", "kernel": "gate_up_mfma_kernel", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
             "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4)}
        r.update(measured_traffic(config_name, r["kernel"], build_id))
        r.update({"algorithmic_bytes_per_launch": ab["gate_up"], "avg_launch_us": round(gu_us, 2)})
        return r
    # prefill-sized batch: 128-row units; the kernel is MFMA bound.  The MFMA takes e2m1 weights and e4m3
    # activations, which issues at the fp8 rate: priced against the fp8 peak
    gu_flops = 2.0 * n * (cfg.topk * cfg.inter + cfg.shared_inter) * 2 * cfg.hidden
    tf = gu_flops / (gu_us * 1e-6) / 1e12
    r = {"bound": "mfma", "kernel": "gate_up_stream_kernel", "achieved": round(tf, 1), "peak": MFMA_PEAK_FP8_TFLOPS,
         "unit": "TFLOP/s", "frac": round(tf / MFMA_PEAK_FP8_TFLOPS, 4)}
    r.update(measured_traffic(config_name, r["kernel"], build_id))
    r.update({"algorithmic_flops_per_launch": gu_flops, "avg_launch_us": round(gu_us, 2),
              "frac_of_fp4_peak": round(tf / MFMA_PEAK_FP4_TFLOPS, 4)})
    return r


def f32_parity(oracle, inp, gpu_rows, ids_gpu, sel, n_threads, ref=None):
    """Distance of the GPU output rows `sel` from the f32 oracle (CpuBackend's arithmetic) on the same inputs."""
    if ref is None:
        ref = oracle.moe_ffn_mxfp4(inp, act_mode=0, n_threads=n_threads, tok_sel=sel)
    d = float(np.abs(gpu_rows.astype(np.float64) - ref["out"]).max() / np.abs(ref["out"]).max())
    return {"max_abs_rel": float(f"{d:.3e}"), "tokens": int(len(sel)),
            "router_ids_equal": bool(np.array_equal(ids_gpu, ref["ids"].astype(np.int32)))}


def decode_step(hip, torch, synth, cfg, n_layers, mode, steps, warmup):
    """The 42-layer decode step (configs[4]): every layer has its own weights, li_0 = x, li_{l+1} = ffn_out_l, every
    layer normalises its input first (rmsnorm -> layer, exec/lib.rs:487-490), one workspace, ONE hipGraph per step."""
    n = cfg.n
    t0 = time.time()
    layers = []
    for li in range(n_layers):
        inp = synth.make_inputs(cfg, seed=0, layer=li)
        layers.append(hip.load_moe_layer(inp, keep_checkpoint_layout=False))
        if li == 0:
            x_in = torch.from_numpy(synth.round_to_bf16(inp.x) if cfg.act_bf16 else inp.x).to(hip.device).float().contiguous()
        del inp
    setup_s = time.time() - t0
    mode = hip.effective_mode(layers[0], n, mode)
    g = torch.Generator(device="cpu").manual_seed(2)
    norm_ws = [(torch.rand(cfg.hidden, generator=g) + 0.5).to(hip.device) for _ in layers]
    ping = [torch.empty(n, cfg.hidden, device=hip.device) for _ in range(2)]
    bws = hip.block_workspace(layers[0], n, mode)

    def step():
        src = x_in
        for i, ly in enumerate(layers):
            dst = ping[i & 1]
            hip.moe_block_mxfp4(ly, src, norm_ws[i], 1e-6, None, None, None, dst, mode, workspace=bws)
            src = dst

    step()
    hip.sync()
    hip.begin_capture()
    step()
    trace = hip.end_capture()
    ms = time_replays(hip, torch, lambda: hip.begin_verify(trace), steps, warmup) * 1e3
    hip.graph_destroy(trace)
    # experts hit in every layer of the chain, from the tables each layer leaves in the shared workspace
    step_bytes, src, hit = 0, x_in, []
    for i, ly in enumerate(layers):
        dst = ping[i & 1]
        hip.moe_block_mxfp4(ly, src, norm_ws[i], 1e-6, None, None, None, dst, mode, workspace=bws)
        hip.sync()
        c = hip.workspace_view(ly, n, mode, workspace=bws)["counts"].cpu().numpy()
        hit.append(int((c > 0).sum()))
        step_bytes += algorithmic_bytes(cfg, n, hit[-1])["total"]
        src = dst
    finite = bool(torch.isfinite(ping[(n_layers - 1) & 1]).all().item())
    return {"workload": WORKLOADS["c4"], "tokens": n, "layers": n_layers, "steps": steps,
            "activation_terms": {1: "fp8", 2: "fp8x2"}[mode],
            "ms_per_step": round(ms, 4), "us_per_layer": round(ms * 1e3 / n_layers, 2),
            "tokens_per_s": round(n / (ms * 1e-3), 1), "step_algorithmic_bytes": step_bytes,
            "step_hbm_gbs": round(step_bytes / (ms * 1e-3) / 1e9, 1),
            "step_hbm_frac": round(step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "experts_hit_min": min(hit), "output_finite": finite, "setup_s": round(setup_s, 1)}, layers, step_bytes


def layer_leg(hip, torch, ev, layer, x, n, cfg, mode, steps, warmup, stack=True):
    """One layer per captured graph: seconds-per-replay timing, the same layer eight times inside one graph, the
    per-stage events and the gate/up kernel's own duration."""
    from ferrite_amd.backend import MODE_MFMA_FP8_X2
    out = torch.empty(n, cfg.hidden, dtype=x.dtype, device=hip.device)
    ws = hip.workspace(layer, n, mode)
    for _ in range(3):
        hip.moe_layer_dev_mxfp4(layer, x, out, mode, ws)
    hip.sync()
    hip.begin_capture()
    hip.moe_layer_dev_mxfp4(layer, x, out, mode, ws)
    trace = hip.end_capture()
    us = time_replays(hip, torch, lambda: hip.begin_verify(trace), steps, warmup) * 1e6
    hip.graph_destroy(trace)
    us_stack = None
    if stack:
        STACK = 8
        hip.begin_capture()
        for _ in range(STACK):
            hip.moe_layer_dev_mxfp4(layer, x, out, mode, ws)
        st = hip.end_capture()
        us_stack = time_replays(hip, torch, lambda: hip.begin_verify(st), max(4, min(50, steps // 4)), 3) / STACK * 1e6
        hip.graph_destroy(st)
    stage_us, eager_us, gu_us = stage_profile(hip, ev, layer, x, out, mode, ws, min(steps, 50))
    gpu_out = out.float().cpu().numpy()
    view = hip.workspace_view(layer, n, mode)
    return dict(us=us, us_stack=us_stack, stage_us=stage_us, eager_us=eager_us, gu_us=gu_us, out=gpu_out,
                ids=view["ids"].cpu().numpy(), counts=view["counts"].cpu().numpy(),
                terms="fp8x2" if mode == MODE_MFMA_FP8_X2 else "fp8")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="c1", choices=sorted(WORKLOADS))
    ap.add_argument("--tokens", type=int, default=0, help="override the token count of the config")
    ap.add_argument("--layers", type=int, default=0,
                    help="chain this many distinct layers into one captured step (default: 42 for c4, else 1)")
    ap.add_argument("--mode", default="auto", choices=["auto", "fp8", "fp8x2"],
                    help="activation format of the expert GEMMs: one e4m3 term, two, or auto = two for decode-sized "
                         "batches and one for prefill-sized ones")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-load-bench", action="store_true",
                    help="skip the checkpoint -> packed-buffer load measurement (writes a shard of the layer to TMPDIR)")
    ap.add_argument("--no-prefill-leg", action="store_true", help="skip the 4096-token leg of the default run")
    ap.add_argument("--no-decode-step-leg", action="store_true",
                    help="skip the 42-layer decode step (54 GB of weights, about a minute of set-up) of the default run")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of graph replays")
    ap.add_argument("--calib-copy-mib", type=int, default=0,
                    help="also run a plain device copy of this many MiB (a counter calibration point for rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    from ferrite_amd import synth
    from ferrite_amd.backend import MODE_MFMA_FP8, MODE_MFMA_FP8_X2, HipBackend

    cfg = synth.CONFIGS[args.config]
    if args.tokens:
        cfg = cfg.with_tokens(args.tokens)
    n = cfg.n
    hip = HipBackend()
    ev = HipEvents()
    n_layers = args.layers or (42 if args.config == "c4" else 1)
    asked = MODE_MFMA_FP8 if args.mode == "fp8" else MODE_MFMA_FP8_X2

    def pick_mode(layer, n):
        """auto: two terms for decode-sized batches (16-row units: the weight stream bounds the call and the second
        term rides on it), the reference's one-term serving format for prefill-sized ones, whose two-term cost is
        reported beside it; a mode the library declines falls back either way."""
        want = asked
        if args.mode == "auto" and hip.unit_rows(layer, n, MODE_MFMA_FP8_X2) != 16:
            want = MODE_MFMA_FP8
        return hip.effective_mode(layer, n, want)
    oracle = None
    if not args.no_cpu_baseline:
        from oracle import binding as oracle

    if args.calib_copy_mib:
        src = torch.ones(args.calib_copy_mib << 20, dtype=torch.uint8, device=hip.device)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- the chained decode step (configs[4]) as the workload of its own ----
    if n_layers > 1:
        step, layers, step_bytes = decode_step(hip, torch, synth, cfg, n_layers, asked, args.steps, args.warmup)
        mode = pick_mode(layers[0], n)
        inp = synth.make_inputs(cfg, seed=0)
        x = torch.from_numpy(inp.x).to(hip.device)
        x = x.to(torch.bfloat16) if cfg.act_bf16 else x
        leg = layer_leg(hip, torch, ev, layers[0], x, n, cfg, mode, min(args.steps, 50), 3, stack=False)
        n_active = int((leg["counts"] > 0).sum())
        ab = algorithmic_bytes(cfg, n, n_active)
        unit_rows = hip.unit_rows(layers[0], n, mode)
        ms = step["ms_per_step"]
        result = {
            "metric": "moe_layer_tokens_per_s", "value": round(n * n_layers / (ms * 1e-3), 1), "unit": "tokens/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "mxfp4 x e4m3 (two terms) -> f32" if mode == MODE_MFMA_FP8_X2 else "mxfp4 x e4m3 -> f32",
            "data": "synthetic",
            "config": {"workload": WORKLOADS[args.config], "tokens": n, "hidden": cfg.hidden, "experts": cfg.n_experts,
                       "topk": cfg.topk, "n_group": cfg.n_group, "topk_group": cfg.topk_group, "inter": cfg.inter,
                       "activation_terms": leg["terms"], "launch": "hipGraph replay", "layers": n_layers,
                       "value_counts": "token-layers per second (tokens x layers / step time)"},
            "layers_per_step": n_layers, "step_algorithmic_bytes": step_bytes, "step_hbm_gbs": step["step_hbm_gbs"],
            "step_hbm_frac": step["step_hbm_frac"], "us_per_layer": step["us_per_layer"],
            "stage_us_one_layer": {k: round(v, 2) for k, v in leg["stage_us"].items()},
            "experts_hit": n_active, "unit_rows": unit_rows, "output_finite": step["output_finite"],
            "roofline": gate_up_roofline(cfg, n, unit_rows, leg["gu_us"], ab, None if args.tokens else args.config,
                                         hip.build_id),
            "cpu_baseline": None, "setup_s": step["setup_s"], "build_id": hip.build_id,
        }
        print(json.dumps(result))
        return

    t0 = time.time()
    inp = synth.make_inputs(cfg, seed=0)
    layer = hip.load_moe_layer(inp, keep_checkpoint_layout=False)
    t_setup = time.time() - t0
    mode = pick_mode(layer, n)
    x = torch.from_numpy(inp.x).to(hip.device)
    if cfg.act_bf16:
        x = x.to(torch.bfloat16)

    if args.no_graph:
        out = torch.empty(n, cfg.hidden, dtype=x.dtype, device=hip.device)
        ws = hip.workspace(layer, n, mode)
        us = time_replays(hip, torch, lambda: hip.moe_layer_dev_mxfp4(layer, x, out, mode, ws), args.steps, args.warmup) * 1e6
        stage_us, eager_us, gu_us = stage_profile(hip, ev, layer, x, out, mode, ws, min(args.steps, 50))
        view = hip.workspace_view(layer, n, mode)
        leg = dict(us=us, us_stack=None, stage_us=stage_us, eager_us=eager_us, gu_us=gu_us, out=out.float().cpu().numpy(),
                   ids=view["ids"].cpu().numpy(), counts=view["counts"].cpu().numpy(),
                   terms="fp8x2" if mode == MODE_MFMA_FP8_X2 else "fp8")
    else:
        leg = layer_leg(hip, torch, ev, layer, x, n, cfg, mode, args.steps, args.warmup)
    ms_per_step = leg["us"] * 1e-3
    counts = leg["counts"]
    n_active = int((counts > 0).sum())
    ab = algorithmic_bytes(cfg, n, n_active)
    flops = 2.0 * n * (cfg.topk * cfg.inter + cfg.shared_inter) * 3 * cfg.hidden
    unit_rows = hip.unit_rows(layer, n, mode)
    roofline = gate_up_roofline(cfg, n, unit_rows, leg["gu_us"], ab, None if args.tokens else args.config, hip.build_id)
    default_run = args.config == "c1" and not args.tokens and not args.no_graph
    ncores = min(16, os.cpu_count() or 1)

    # the reference's own serving format beside the two-term one: same layer, one e4m3 term (quant.rs:201-214)
    decode_fp8 = None
    if default_run and mode == MODE_MFMA_FP8_X2:
        l1 = layer_leg(hip, torch, ev, layer, x, n, cfg, MODE_MFMA_FP8, max(20, args.steps // 2), 5)
        decode_fp8 = {"activation_terms": "fp8", "us_per_layer": round(l1["us"], 2),
                      "us_per_layer_in_stack": round(l1["us_stack"], 2),
                      "gate_up_kernel_us": round(l1["gu_us"], 2),
                      "layer_hbm_frac": round(ab["total"] / (l1["us"] * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                      "what": "the same layer with one e4m3 term per activation, the reference's serving format"}
        if oracle is not None:
            decode_fp8["parity_vs_f32_oracle"] = f32_parity(oracle, inp, l1["out"][:min(n, 32)], l1["ids"],
                                                            np.arange(min(n, 32), dtype=np.int32), ncores)

    # the FFN half of a decoder layer around the same layer (exec/lib.rs:487-492): rmsnorm -> layer -> hc_post as one
    # captured call, and the two neighbours on their own (torch events on the backend's stream)
    block = None
    if not args.no_graph:
        nh = 4
        g = torch.Generator(device="cpu").manual_seed(1)
        li = (torch.randn(n, cfg.hidden, generator=g) * 3.0).to(hip.device)
        norm_w = (torch.rand(cfg.hidden, generator=g) + 0.5).to(hip.device)
        residual = torch.randn(n, nh, cfg.hidden, generator=g).to(hip.device)
        post = (torch.rand(n, nh, generator=g) * 2.0).to(hip.device)
        comb = torch.softmax(torch.randn(n, nh, nh, generator=g), dim=2).to(hip.device)
        bout = torch.empty(n, nh, cfg.hidden, device=hip.device)
        hfn = torch.empty(n, cfg.hidden, device=hip.device)
        for _ in range(3):
            hip.moe_block_mxfp4(layer, li, norm_w, 1e-6, residual, post, comb, bout, mode)
        hip.sync()
        hip.begin_capture()
        hip.moe_block_mxfp4(layer, li, norm_w, 1e-6, residual, post, comb, bout, mode)
        btrace = hip.end_capture()
        us_block = time_replays(hip, torch, lambda: hip.begin_verify(btrace), max(10, min(200, args.steps)), 3) * 1e6
        hip.graph_destroy(btrace)

        def op_us(fn):
            with torch.cuda.stream(hip.stream):
                for _ in range(5):
                    fn()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(hip.stream)
                for _ in range(50):
                    fn()
                e1.record(hip.stream)
            e1.synchronize()
            return e0.elapsed_time(e1) / 50 * 1e3

        block = {"us_per_block": round(us_block, 2), "hc_streams": nh,
                 "rmsnorm_us": round(op_us(lambda: hip.rmsnorm(li, norm_w, 1e-6, hfn)), 2),
                 "hc_post_us": round(op_us(lambda: hip.hc_post(hfn, residual, post, comb)), 2)}
        del li, residual, bout, hfn

    # the other half of the metric on the same weights: the 4096-token prefill chunk (c2 is c1's layer at n = 4096).
    # Asked for in the same mode as the decode leg: the library declines two terms at this size and the backend falls
    # back to one e4m3 term, the format that configuration prescribes
    prefill = None
    if default_run and not args.no_prefill_leg:
        pcfg = synth.CONFIGS["c2"]
        pn = pcfg.n
        px_np = synth.make_activations(pcfg, seed=0)
        px = torch.from_numpy(px_np).to(hip.device).to(torch.bfloat16)
        pmode = pick_mode(layer, pn)
        pl = layer_leg(hip, torch, ev, layer, px, pn, pcfg, pmode, max(10, min(50, args.steps)), 20, stack=False)
        pcounts = pl["counts"]
        pab = algorithmic_bytes(pcfg, pn, int((pcounts > 0).sum()))
        pflops = 2.0 * pn * (pcfg.topk * pcfg.inter + pcfg.shared_inter) * 3 * pcfg.hidden
        ptf = pflops / (pl["us"] * 1e-6) / 1e12
        prefill = {"workload": WORKLOADS["c2"], "tokens": pn, "steps": max(10, min(50, args.steps)),
                   "activation_terms": pl["terms"], "us_per_layer": round(pl["us"], 2),
                   "tokens_per_s": round(pn / (pl["us"] * 1e-6), 1), "layer_tflops": round(ptf, 1),
                   "mfma_frac_of_fp8_peak": round(ptf / MFMA_PEAK_FP8_TFLOPS, 4),
                   "mfma_frac_of_mxfp4_peak": round(ptf / MFMA_PEAK_FP4_TFLOPS, 4),
                   "stage_us": {k: round(v, 2) for k, v in pl["stage_us"].items()},
                   "max_over_mean_tokens_per_expert": round(float(pcounts.max() / max(pcounts.mean(), 1e-9)), 2),
                   "roofline": gate_up_roofline(pcfg, pn, hip.unit_rows(layer, pn, pmode), pl["gu_us"], pab, "c2",
                                                hip.build_id)}
        if oracle is not None:
            # the same 32-token sample the CPU baseline takes: evenly spaced tokens of the chunk, routed on the CPU too
            import dataclasses
            sel = np.linspace(0, pn - 1, 32).astype(np.int32)
            pinp = dataclasses.replace(inp, cfg=pcfg, x=synth.round_to_bf16(px_np))
            pref = oracle.moe_ffn_mxfp4(pinp, act_mode=0, n_threads=ncores, tok_sel=sel)
            prefill["parity_vs_f32_oracle"] = f32_parity(oracle, pinp, pl["out"][sel], pl["ids"], sel, ncores, pref)
            prefill["parity_vs_f32_oracle"]["what"] = ("one e4m3 term per activation (three mantissa bits) against the "
                                                       "unquantised f32 oracle; router ids compared for all tokens")
            del pinp
        # the same chunk with two e4m3 terms per activation (64-row units): what the 2e-2 bar costs at prefill
        from ferrite_amd.backend import MODE_MFMA_FP8_X2 as _X2
        pl2 = layer_leg(hip, torch, ev, layer, px, pn, pcfg, _X2, max(10, min(30, args.steps)), 10, stack=False)
        prefill["two_term"] = {"activation_terms": pl2["terms"], "unit_rows": hip.unit_rows(layer, pn, _X2),
                               "us_per_layer": round(pl2["us"], 2),
                               "tokens_per_s": round(pn / (pl2["us"] * 1e-6), 1),
                               "stage_us": {k: round(v, 2) for k, v in pl2["stage_us"].items()},
                               "gate_up_kernel_us": round(pl2["gu_us"], 2),
                               "what": "both planes of x and of the SwiGLU output, a second MFMA per tile against the "
                                       "same weight registers: twice the MFMAs and fills of the one-term chunk"}
        if oracle is not None:
            prefill["two_term"]["parity_vs_f32_oracle"] = f32_parity(oracle, None, pl2["out"][sel], pl2["ids"], sel, ncores, pref)
        del px, pl, pl2

    # the row before the layer: one layer's shard (safetensors, the reference's tensor names) streamed from the
    # page cache into the packed buffer; PCIe-bound, priced against a pinned -> device copy of the same size
    load = None
    if not args.no_load_bench:
        try:
            import tempfile
            from ferrite_amd import checkpoint as ckpt
            with tempfile.TemporaryDirectory() as td:
                shard = os.path.join(td, "layer.safetensors")
                ckpt.write_moe_checkpoint(shard, inp, "layers.6.ffn", ckpt.NAMING_DSV41)
                with ckpt.Checkpoint(shard) as c:
                    runs = []
                    for _ in range(4):
                        loaded, st = c.load_moe_layer(hip, cfg, "layers.6.ffn", ckpt.NAMING_DSV41)
                        runs.append(st)
                    same = bool(torch.equal(loaded.packed, layer.packed))
                    del loaded
                best = min(runs[1:], key=lambda r: r.seconds)
                pin = torch.empty(best.source_bytes, dtype=torch.uint8).pin_memory()
                dst = torch.empty(best.source_bytes, dtype=torch.uint8, device=hip.device)
                copy_s = []
                for _ in range(3):
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    dst.copy_(pin, non_blocking=True)
                    torch.cuda.synchronize()
                    copy_s.append(time.perf_counter() - t0)
                del pin, dst
                pcie = best.source_bytes / min(copy_s) / 1e9
                load = {"source_bytes": best.source_bytes, "workers": best.workers,
                        "first_load_ms": round(runs[0].seconds * 1e3, 2), "ms": round(best.seconds * 1e3, 2),
                        "GB_per_s": round(best.source_bytes / best.seconds / 1e9, 2),
                        "pinned_copy_GB_per_s": round(pcie, 2),
                        "frac_of_pinned_copy": round(best.source_bytes / best.seconds / 1e9 / pcie, 4),
                        "packed_equals_memory_loaded": same,
                        "what": "safetensors shard in the page cache -> pinned staging -> device -> repack kernels; "
                                "first load also allocates the staging buffers"}
        except Exception as e:   # a full TMPDIR must not cost the layer's numbers
            load = {"error": f"{type(e).__name__}: {e}"}

    cpu, parity = None, None
    if oracle is not None:
        # the whole layer for a bounded token sample, single thread (the reference's CpuBackend is
        # single-threaded scalar code), f32 activations as CpuBackend computes
        ns = min(n, 32)
        sel = np.linspace(0, n - 1, ns).astype(np.int32)
        reps = 0
        t0 = time.perf_counter()
        while True:
            ref = oracle.moe_ffn_mxfp4(inp, act_mode=0, n_threads=1, tok_sel=sel)
            reps += 1
            if time.perf_counter() - t0 > 12.0 or reps >= 12:
                break
        t1 = (time.perf_counter() - t0) / reps
        t0 = time.perf_counter()
        oracle.moe_ffn_mxfp4(inp, act_mode=0, n_threads=ncores, tok_sel=sel)
        tall = time.perf_counter() - t0
        extrap = "" if ns == n else (f"; the whole batch of {n} tokens would take {t1 * n / ns:.0f} s at this rate "
                                     "(linear extrapolation, not measured)")
        cpu = {"value": round(ns / t1, 2), "unit": "tokens/s", "cores": 1, "kind": "port",
               "sample": f"full layer (routing of all {n} tokens + experts + shared + combine) for {ns} tokens, "
                         f"{reps} repetition(s), {t1:.2f} s each, f32 activations" + extrap,
               "all_cores": {"value": round(ns / tall, 2), "cores": ncores, "seconds": round(tall, 2)}}
        # the same run is the parity check of this process's GPU output: the f32 oracle is CpuBackend's arithmetic
        ids_equal = bool(np.array_equal(leg["ids"], ref["ids"].astype(np.int32)))
        d = float(np.abs(leg["out"][sel].astype(np.float64) - ref["out"]).max() / np.abs(ref["out"]).max())
        parity = {"max_abs_rel": float(f"{d:.3e}"), "tokens": ns, "router_ids_equal": ids_equal,
                  "what": "max|gpu - oracle| / max|oracle| of the layer output over the sampled tokens, oracle = the f32 "
                          "CPU restatement of CpuBackend (act_mode 0); output rounded to bf16 where the config says so"}

    # the 42-layer decode step of configs[4] (192 tokens) as one hipGraph: last, it needs 54 GB for its weights
    dstep = None
    if default_run and not args.no_decode_step_leg:
        del layer
        torch.cuda.empty_cache()
        dstep, dlayers, _ = decode_step(hip, torch, synth, synth.CONFIGS["c4"], 42, asked,
                                        max(5, min(50, args.steps)), 2)
        del dlayers

    us_layer = leg["us"]
    result = {
        "metric": "moe_layer_tokens_per_s", "value": round(n / (ms_per_step * 1e-3), 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "mxfp4 x e4m3 (two terms) -> f32" if mode == MODE_MFMA_FP8_X2 else "mxfp4 x e4m3 -> f32",
        "data": "synthetic",
        "config": {"workload": WORKLOADS[args.config], "tokens": n, "hidden": cfg.hidden, "experts": cfg.n_experts,
                   "topk": cfg.topk, "n_group": cfg.n_group, "topk_group": cfg.topk_group, "inter": cfg.inter,
                   "activation_terms": leg["terms"],
                   "activation_format_note": "two e4m3 terms per activation is this build's own format (no reference "
                                             "fixture); the reference's one-term format is timed under decode_fp8"
                   if mode == MODE_MFMA_FP8_X2 else "one e4m3 term per activation, the reference's serving format",
                   "launch": "eager" if args.no_graph else "hipGraph replay"},
        "layers_per_step": 1, "step_algorithmic_bytes": ab["total"],
        "step_hbm_gbs": round(ab["total"] / (ms_per_step * 1e-3) / 1e9, 1),
        "us_per_layer": round(us_layer, 2), "us_per_layer_eager_events": round(leg["eager_us"], 2),
        "us_per_layer_in_stack": None if leg["us_stack"] is None else round(leg["us_stack"], 2),
        "stage_us": {k: round(v, 2) for k, v in leg["stage_us"].items()},
        "experts_hit": n_active, "max_tokens_per_expert": int(counts.max()),
        "max_over_mean_tokens_per_expert": round(float(counts.max() / max(counts.mean(), 1e-9)), 2),
        "layer_algorithmic_bytes": ab["total"],
        "layer_hbm_gbs": round(ab["total"] / (us_layer * 1e-6) / 1e9, 1),
        "layer_hbm_frac": round(ab["total"] / (us_layer * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
        "layer_tflops": round(flops / (us_layer * 1e-6) / 1e12, 2),
        "mfma_frac_of_fp8_peak": round(flops / (us_layer * 1e-6) / 1e12 / MFMA_PEAK_FP8_TFLOPS, 4),
        "mfma_frac_of_mxfp4_peak": round(flops / (us_layer * 1e-6) / 1e12 / MFMA_PEAK_FP4_TFLOPS, 4),
        "parity_vs_f32_oracle": parity, "decode_fp8": decode_fp8, "prefill": prefill, "decode_step": dstep,
        "block_rmsnorm_layer_hc_post": block, "checkpoint_load": load, "unit_rows": unit_rows, "roofline": roofline,
        "cpu_baseline": cpu, "setup_s": round(t_setup, 1), "build_id": hip.build_id,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
