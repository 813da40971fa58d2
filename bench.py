#!/usr/bin/env python3
"""Benchmark of the MoE FFN layer on one MI355X.

One "step" = one pass of the fused layer (router GEMM -> routing -> permutation -> activation quantisation ->
gate/up GEMM + SwiGLU -> down GEMM -> combine) over one batch of synthetic tokens, replayed from a captured
hipGraph the way a decode step runs in production.  Inputs and weights are resident in HBM before the timed
region.  Prints ONE JSON line (see README / DESIGN for the fields).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c1] [--no-cpu-baseline]

The default run times the decode layer (c1: 32 tokens) and, on the same weights, a bounded prefill leg (c2: 4096
tokens) reported under "prefill".  --config c4 runs the 42-layer decode step: every layer has its own weights, the
layers are chained (rmsnorm of a layer's output is the next layer's input) and share one workspace, and the whole
step is one hipGraph.
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
# are in profiles/.  Counters cannot be read inside this script.
MEASURED_TRAFFIC = {("c1", "gate_up_mfma_kernel"): 764.6e6, ("c2", "gate_up_prefill_kernel"): 1470.3e6}

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


def gate_up_roofline(cfg, n, unit_rows, gu_us, ab, traffic_key):
    if unit_rows != 128:
        # decode-sized batch: every weight byte is streamed once per unit; the kernel is HBM bound
        gbs = ab["gate_up"] / (gu_us * 1e-6) / 1e9
        return {"bound": "hbm", "kernel": "gate_up_mfma_kernel", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC.get(traffic_key),
                "algorithmic_bytes_per_launch": ab["gate_up"], "avg_launch_us": round(gu_us, 2)}
    # prefill-sized batch: 128-row units, both operands tiled through LDS; the kernel is MFMA bound.  The MFMA takes
    # e2m1 weights and e4m3 activations, which issues at the fp8 rate: priced against the fp8 peak
    gu_flops = 2.0 * n * (cfg.topk * cfg.inter + cfg.shared_inter) * 2 * cfg.hidden
    tf = gu_flops / (gu_us * 1e-6) / 1e12
    return {"bound": "mfma", "kernel": "gate_up_prefill_kernel", "achieved": round(tf, 1), "peak": MFMA_PEAK_FP8_TFLOPS,
            "unit": "TFLOP/s", "frac": round(tf / MFMA_PEAK_FP8_TFLOPS, 4), "traffic": MEASURED_TRAFFIC.get(traffic_key),
            "algorithmic_flops_per_launch": gu_flops, "avg_launch_us": round(gu_us, 2),
            "frac_of_fp4_peak": round(tf / MFMA_PEAK_FP4_TFLOPS, 4)}


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
                    help="activation format of the expert GEMMs: one e4m3 term, two (decode-sized batches only), or "
                         "auto = two where they are supported")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-load-bench", action="store_true",
                    help="skip the checkpoint -> packed-buffer load measurement (writes a shard of the layer to TMPDIR)")
    ap.add_argument("--no-prefill-leg", action="store_true", help="skip the 4096-token leg of the default run")
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
    n_layers = args.layers or (42 if args.config == "c4" else 1)
    decode_sized = n * cfg.topk < 48 * cfg.n_experts
    if args.mode == "fp8x2" and not decode_sized:
        print("--mode fp8x2 is for decode-sized batches (n*topk < 48*experts)", file=sys.stderr)
        sys.exit(2)
    mode = MODE_MFMA_FP8_X2 if (args.mode == "fp8x2" or (args.mode == "auto" and decode_sized)) else MODE_MFMA_FP8
    mode_name = {MODE_MFMA_FP8: "fp8", MODE_MFMA_FP8_X2: "fp8x2"}[mode]
    t0 = time.time()
    inp = synth.make_inputs(cfg, seed=0)
    layer = hip.load_moe_layer(inp, keep_checkpoint_layout=False)
    layers = [layer]
    for li in range(1, n_layers):
        extra = synth.make_inputs(cfg, seed=0, layer=li)
        layers.append(hip.load_moe_layer(extra, keep_checkpoint_layout=False))
        del extra
    t_setup = time.time() - t0

    x = torch.from_numpy(inp.x).to(hip.device)
    if cfg.act_bf16:
        x = x.to(torch.bfloat16)
    out = torch.empty(n, cfg.hidden, dtype=x.dtype, device=hip.device)
    ws = hip.workspace(layer, n, mode)

    if n_layers == 1:
        def step():
            hip.moe_layer_dev_mxfp4(layer, x, out, mode, ws)
    else:
        # The chained step: li_0 = x; li_{l+1} = ffn_out_l; every layer normalises its input first (rmsnorm ->
        # layer, exec/lib.rs:487-490), which keeps the activations, and with them the routing, at their scale through
        # all layers.  One workspace; the input buffer is never written, so replays start from the same data.
        g = torch.Generator(device="cpu").manual_seed(2)
        norm_ws = [(torch.rand(cfg.hidden, generator=g) + 0.5).to(hip.device) for _ in layers]
        x_in = x.float().contiguous()
        ping = [torch.empty(n, cfg.hidden, device=hip.device) for _ in range(2)]
        bws = hip.block_workspace(layer, n, mode)

        def step():
            src = x_in
            for i, ly in enumerate(layers):
                dst = ping[i & 1]
                hip.moe_block_mxfp4(ly, src, norm_ws[i], 1e-6, None, None, None, dst, mode, workspace=bws)
                src = dst

    if args.calib_copy_mib:
        src = torch.ones(args.calib_copy_mib << 20, dtype=torch.uint8, device=hip.device)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # warm up eagerly (fills caches), then capture one step as a graph
    for _ in range(max(min(args.warmup, 5), 2)):
        step()
    hip.sync()
    trace = None
    if not args.no_graph:
        hip.begin_capture()
        step()
        trace = hip.end_capture()
    replay = step if trace is None else (lambda: hip.begin_verify(trace))
    ms_per_step = time_replays(hip, torch, replay, args.steps, args.warmup) * 1e3

    # A graph launch costs about 13 us on the device before its first kernel starts; a model runs all its layers
    # from one graph, so the same layer is also timed eight times back to back inside one graph (reported as
    # us_per_layer_in_stack; `value` stays the single-layer-per-launch figure).
    us_in_stack = None
    if trace is not None and n_layers == 1:
        STACK = 8
        hip.begin_capture()
        for _ in range(STACK):
            step()
        stack_trace = hip.end_capture()
        reps = max(4, min(50, args.steps // 4))
        us_in_stack = time_replays(hip, torch, lambda: hip.begin_verify(stack_trace), reps, 3) / STACK * 1e6
        hip.graph_destroy(stack_trace)

    # The FFN half of a decoder layer around the same layer (exec/lib.rs:487-492): rmsnorm -> layer -> hc_post as one
    # captured call, and the two neighbours on their own (torch events on the backend's stream).
    block = None
    if trace is not None and n_layers == 1:
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

    ev = HipEvents()
    stage_us, eager_us, gu_kernel_us = stage_profile(hip, ev, layer, x, out, mode, ws, min(args.steps, 50))
    gpu_out = out.float().cpu().numpy()      # layer 0 on the config's own input (the eager passes just above)

    view = hip.workspace_view(layer, n, mode)
    counts = view["counts"].cpu().numpy()
    n_active = int((counts > 0).sum())
    ab = algorithmic_bytes(cfg, n, n_active)
    step_bytes = ab["total"] * n_layers
    if n_layers > 1:
        # experts hit in every layer of the chain, from the tables each layer leaves in the shared workspace
        step_bytes, src = 0, x_in
        for i, ly in enumerate(layers):
            dst = ping[i & 1]
            hip.moe_block_mxfp4(ly, src, norm_ws[i], 1e-6, None, None, None, dst, mode, workspace=bws)
            hip.sync()
            c = hip.workspace_view(ly, n, mode, workspace=bws)["counts"].cpu().numpy()
            step_bytes += algorithmic_bytes(cfg, n, int((c > 0).sum()))["total"]
            src = dst
    flops = 2.0 * n * (cfg.topk * cfg.inter + cfg.shared_inter) * 3 * cfg.hidden

    us_layer = ms_per_step * 1e3 / n_layers
    unit_rows = hip.unit_rows(layer, n, mode)
    kname = "gate_up_prefill_kernel" if unit_rows == 128 else "gate_up_mfma_kernel"
    roofline = gate_up_roofline(cfg, n, unit_rows, gu_kernel_us, ab, None if args.tokens else (args.config, kname))

    # the other half of the metric on the same weights: the 4096-token prefill chunk (c2 is c1's layer at n = 4096),
    # one e4m3 term as that configuration prescribes; a bounded number of replays
    prefill = None
    if args.config == "c1" and not args.tokens and not args.no_prefill_leg and trace is not None:
        pcfg = synth.CONFIGS["c2"]
        pn = pcfg.n
        px = torch.from_numpy(synth.make_activations(pcfg, seed=0)).to(hip.device).to(torch.bfloat16)
        pout = torch.empty(pn, pcfg.hidden, dtype=torch.bfloat16, device=hip.device)
        pws = hip.workspace(layer, pn, MODE_MFMA_FP8)
        for _ in range(3):
            hip.moe_layer_dev_mxfp4(layer, px, pout, MODE_MFMA_FP8, pws)
        hip.sync()
        hip.begin_capture()
        hip.moe_layer_dev_mxfp4(layer, px, pout, MODE_MFMA_FP8, pws)
        ptrace = hip.end_capture()
        p_steps = max(10, min(50, args.steps))
        p_us = time_replays(hip, torch, lambda: hip.begin_verify(ptrace), p_steps, 5) * 1e6
        hip.graph_destroy(ptrace)
        p_stage, _, p_gu_us = stage_profile(hip, ev, layer, px, pout, MODE_MFMA_FP8, pws, 10)
        pcounts = hip.workspace_view(layer, pn, MODE_MFMA_FP8)["counts"].cpu().numpy()
        pab = algorithmic_bytes(pcfg, pn, int((pcounts > 0).sum()))
        pflops = 2.0 * pn * (pcfg.topk * pcfg.inter + pcfg.shared_inter) * 3 * pcfg.hidden
        ptf = pflops / (p_us * 1e-6) / 1e12
        prefill = {"workload": WORKLOADS["c2"], "tokens": pn, "steps": p_steps, "us_per_layer": round(p_us, 2),
                   "tokens_per_s": round(pn / (p_us * 1e-6), 1), "layer_tflops": round(ptf, 1),
                   "mfma_frac_of_fp8_peak": round(ptf / MFMA_PEAK_FP8_TFLOPS, 4),
                   "mfma_frac_of_mxfp4_peak": round(ptf / MFMA_PEAK_FP4_TFLOPS, 4),
                   "stage_us": {k: round(v, 2) for k, v in p_stage.items()},
                   "max_over_mean_tokens_per_expert": round(float(pcounts.max() / max(pcounts.mean(), 1e-9)), 2),
                   "roofline": gate_up_roofline(pcfg, pn, hip.unit_rows(layer, pn, MODE_MFMA_FP8), p_gu_us, pab,
                                                ("c2", "gate_up_prefill_kernel"))}
        del px, pout

    # the row before the layer: one layer's shard (safetensors, the reference's tensor names) streamed from the
    # page cache into the packed buffer; PCIe-bound, priced against a pinned -> device copy of the same size
    load = None
    if not args.no_load_bench and n_layers == 1:
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
    if not args.no_cpu_baseline:
        from oracle import binding as oracle
        # the whole layer for a bounded token sample, single thread (the reference's CpuBackend is
        # single-threaded scalar code), f32 activations as CpuBackend computes
        ns = min(n, 32)
        sel = np.arange(ns, dtype=np.int32)
        reps = 0
        t0 = time.perf_counter()
        while True:
            ref = oracle.moe_ffn_mxfp4(inp, act_mode=0, n_threads=1, tok_sel=sel)
            reps += 1
            if time.perf_counter() - t0 > 12.0 or reps >= 12:
                break
        t1 = (time.perf_counter() - t0) / reps
        ncores = min(16, os.cpu_count() or 1)
        t0 = time.perf_counter()
        oracle.moe_ffn_mxfp4(inp, act_mode=0, n_threads=ncores, tok_sel=sel)
        tall = time.perf_counter() - t0
        cpu = {"value": round(ns / t1, 2), "unit": "tokens/s", "cores": 1, "kind": "port",
               "sample": f"full layer (routing of all {n} tokens + experts + shared + combine) for {ns} tokens, "
                         f"{reps} repetition(s), {t1:.2f} s each, f32 activations",
               "all_cores": {"value": round(ns / tall, 2), "cores": ncores, "seconds": round(tall, 2)}}
        # the same run is the parity check of this process's GPU output: the f32 oracle is CpuBackend's arithmetic
        ids_equal = bool(np.array_equal(view["ids"].cpu().numpy(), ref["ids"].astype(np.int32)))
        d = float(np.abs(gpu_out[:ns].astype(np.float64) - ref["out"]).max() / np.abs(ref["out"]).max())
        parity = {"max_abs_rel": float(f"{d:.3e}"), "tokens": ns, "router_ids_equal": ids_equal,
                  "what": "max|gpu - oracle| / max|oracle| of the layer output over the sampled tokens, oracle = the f32 "
                          "CPU restatement of CpuBackend (act_mode 0); output rounded to bf16 where the config says so"}

    result = {
        "metric": "moe_layer_tokens_per_s", "value": round(n / (ms_per_step * 1e-3), 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "mxfp4 x e4m3 (two terms) -> f32" if mode == MODE_MFMA_FP8_X2 else "mxfp4 x e4m3 -> f32",
        "data": "synthetic",
        "config": {"workload": WORKLOADS[args.config], "tokens": n, "hidden": cfg.hidden, "experts": cfg.n_experts,
                   "topk": cfg.topk, "n_group": cfg.n_group, "topk_group": cfg.topk_group, "inter": cfg.inter,
                   "activation_terms": mode_name, "launch": "eager" if trace is None else "hipGraph replay"},
        "layers_per_step": n_layers, "step_algorithmic_bytes": step_bytes,
        "step_hbm_gbs": round(step_bytes / (ms_per_step * 1e-3) / 1e9, 1),
        "us_per_layer": round(us_layer, 2), "us_per_layer_eager_events": round(eager_us, 2),
        "us_per_layer_in_stack": None if us_in_stack is None else round(us_in_stack, 2),
        "stage_us": {k: round(v, 2) for k, v in stage_us.items()},
        "experts_hit": n_active, "max_tokens_per_expert": int(counts.max()),
        "max_over_mean_tokens_per_expert": round(float(counts.max() / max(counts.mean(), 1e-9)), 2),
        "layer_algorithmic_bytes": ab["total"],
        "layer_hbm_gbs": round(step_bytes / n_layers / (us_layer * 1e-6) / 1e9, 1),
        "layer_hbm_frac": round(step_bytes / n_layers / (us_layer * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
        "layer_tflops": round(flops / (us_layer * 1e-6) / 1e12, 2),
        "mfma_frac_of_fp8_peak": round(flops / (us_layer * 1e-6) / 1e12 / MFMA_PEAK_FP8_TFLOPS, 4),
        "mfma_frac_of_mxfp4_peak": round(flops / (us_layer * 1e-6) / 1e12 / MFMA_PEAK_FP4_TFLOPS, 4),
        "parity_vs_f32_oracle": parity, "prefill": prefill,
        "block_rmsnorm_layer_hc_post": block, "checkpoint_load": load, "unit_rows": unit_rows, "roofline": roofline,
        "cpu_baseline": cpu, "setup_s": round(t_setup, 1), "build_id": hip.build_id,
    }
    if trace is not None:
        hip.graph_destroy(trace)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
