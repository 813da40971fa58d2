"""Writes the committed golden vectors from the CPU oracle (run from the repo root:
`python tests/golden/make_golden.py`).  Inputs come from the seeded generator, so only outputs are stored."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from ferrite_amd import synth  # noqa: E402
from oracle import binding as oracle  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    inp = synth.make_inputs(synth.CONFIGS["c0"], seed=0)
    f32 = oracle.moe_ffn_mxfp4(inp, act_mode=0)
    fp8 = oracle.moe_ffn_mxfp4(inp, act_mode=1)
    fp8x2 = oracle.moe_ffn_mxfp4(inp, act_mode=2)
    ids = f32["ids"].astype(np.int32)
    t = oracle.moe_permute(ids, inp.cfg.n_experts)
    np.savez_compressed(os.path.join(HERE, "c0_layer.npz"), ids=ids, probs=f32["probs"], logits=f32["logits"],
                        out_f32=f32["out"], out_fp8act=fp8["out"], out_fp8x2=fp8x2["out"], counts=t["counts"], starts=t["starts"],
                        perm_map=t["perm_map"], gather_src=t["gather_src"],
                        x_head=inp.x[0, :8], gate_w_head=inp.gate_w[0, 0, :8], gate_s_head=inp.gate_s[0, 0, :4])
    # format sweep tables: e4m3 decode of all 256 bytes, e2m1 table, e4m3 encode of a fixed ramp
    ramp = (np.arange(-2048, 2048, dtype=np.float32) * np.float32(0.2371)).astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "format_tables.npz"),
                        e4m3_decode=np.array([oracle.e4m3_decode(i) for i in range(256)], np.float32),
                        e2m1_decode=np.array([oracle.e2m1_decode(i) for i in range(16)], np.float32),
                        e4m3_encode_ramp=np.array([oracle.e4m3_encode(float(v)) for v in ramp], np.uint8))


if __name__ == "__main__":
    main()
