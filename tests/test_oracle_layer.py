"""The oracle's layer composition (crates/ferrite-exec/src/lib.rs:1083-1166) against
 (a) the complete small fixture of crates/ferrite-kernel/tests/gpu_smoke.rs:437-562, whose weights are exactly
     representable in MXFP4, evaluated by an independent float64 NumPy statement of the test's algorithm;
 (b) the same float64 statement on the seeded tiny config; (c) the committed golden vectors."""
import os

import numpy as np
import pytest

from ferrite_amd import synth
from tests import refmath


def smoke_fixture():
    """gpu_smoke.rs:437-470: H 64, I 32, Is 16, E 8, k 2, values ((i+s)%4)*0.25-0.5, scale 1.2, limit 7."""
    H, I, Is, E, K = 64, 32, 16, 8, 2
    bex = lambda i, s: ((i + s) % 4) * 0.25 - 0.5
    x = np.array([bex(i, 0) for i in range(H)], np.float32)[None, :]
    gate_w = np.array([bex(i, 5) for i in range(E * H)], np.float32).reshape(E, H)
    bias = np.array([bex(i, 2) for i in range(E)], np.float32)
    mk = lambda r, c, s: np.array([bex(i * 7 + s, 0) for i in range(r * c)], np.float64).reshape(r, c)
    eg = np.stack([mk(I, H, s * 11) for s in range(E)])
    eu = np.stack([mk(I, H, s * 13 + 3) for s in range(E)])
    ed = np.stack([mk(H, I, s * 17 + 7) for s in range(E)])
    sg, su, sd = mk(Is, H, 29), mk(Is, H, 31), mk(H, Is, 37)
    # the shared expert is 16 wide; MXFP4 blocks are 32 wide, so pad it with zero rows/columns (exact no-op)
    sgp = np.zeros((32, H)); sgp[:Is] = sg
    sup = np.zeros((32, H)); sup[:Is] = su
    sdp = np.zeros((H, 32)); sdp[:, :Is] = sd
    cfg = synth.MoeConfig(1, H, E, K, I, 32, 1, 1, routed_scaling=1.2, swiglu_limit=7.0)
    enc = lambda m: refmath.encode_exact(m, 125)   # {-0.5,-0.25,0,0.25} = {-2,-1,0,1} * 2^-2
    gw, gs = enc(eg); uw, us = enc(eu); dw, ds = enc(ed)
    sgw, sgs = enc(sgp[None]); suw, sus = enc(sup[None]); sdw, sds = enc(sdp[None])
    inp = synth.MoeInputs(cfg, x, gate_w, bias, gw, gs, uw, us, dw, ds, sgw, sgs, suw, sus, sdw, sds)
    return inp, (eg, eu, ed, sg, su, sd)


def test_layer_matches_gpu_smoke_fixture_in_float64(oracle):
    inp, (eg, eu, ed, sg, su, sd) = smoke_fixture()
    got = oracle.moe_ffn_mxfp4(inp)
    # the reference algorithm of gpu_smoke.rs:493-562 in float64, on the un-encoded weights
    x = inp.x[0].astype(np.float64)
    logits = inp.router_w.astype(np.float64) @ x
    scores = 1.0 / (1.0 + np.exp(-logits))
    choice = scores + inp.router_bias
    order = sorted(range(8), key=lambda j: -choice[j])[:2]
    probs = scores[order] / scores[order].sum() * 1.2
    silu = lambda g: g / (1.0 + np.exp(-g))
    ref = np.zeros(64)
    for jj, e in enumerate(order):
        g = np.minimum(eg[e] @ x, 7.0)
        u = np.clip(eu[e] @ x, -7.0, 7.0)
        ref += probs[jj] * (ed[e] @ (silu(g) * u))
    g = np.minimum(sg @ x, 7.0)
    u = np.clip(su @ x, -7.0, 7.0)
    ref += sd @ (silu(g) * u)
    assert got["ids"][0].astype(int).tolist() == order
    assert np.allclose(got["probs"][0], probs, atol=1e-6)
    assert np.abs(got["out"][0] - ref).max() < 1e-5
    assert np.abs(ref).max() > 0.1   # the fixture is not degenerate


@pytest.mark.parametrize("grouped", [False, True])
def test_layer_c0_matches_float64_statement(oracle, grouped):
    cfg = synth.CONFIGS["c0"]
    if not grouped:
        cfg = synth.MoeConfig(**{**cfg.__dict__, "n_group": 1, "topk_group": 1})
    inp = synth.make_inputs(cfg, seed=0)
    got = oracle.moe_ffn_mxfp4(inp)
    ref, probs, ids = refmath.moe_layer(inp)
    assert np.array_equal(got["ids"].astype(int), ids)
    assert np.allclose(got["probs"], probs, atol=1e-6)
    assert refmath.max_abs_rel(got["out"], ref) < 1e-5
    # thread count must not change a single bit (parallelism is over tokens/rows only)
    got4 = oracle.moe_ffn_mxfp4(inp, n_threads=4)
    assert np.array_equal(got4["out"], got["out"])


def test_layer_token_subset_equals_full(oracle):
    inp = synth.make_inputs(synth.CONFIGS["c0"], seed=1)
    full = oracle.moe_ffn_mxfp4(inp)
    sub = oracle.moe_ffn_mxfp4(inp, tok_sel=[6, 1, 3])
    assert np.array_equal(sub["out"], full["out"][[6, 1, 3]])
    assert np.array_equal(sub["ids"], full["ids"])


def _layer_cases():
    c0 = synth.CONFIGS["c0"]
    ragged = synth.MoeConfig(13, 384, 8, 3, 256, 128, 4, 2)      # blocks that do not line up with anything
    return [(c0, 0), (c0, 2), (ragged, 5)]


@pytest.mark.parametrize("cfg,seed", _layer_cases())
def test_layer_quantised_activation_modes_match_an_independent_statement(oracle, cfg, seed):
    """act_mode 1 / 2 of the oracle against a NumPy statement that shares nothing with it: float64 GEMMs,
    torch.float8_e4m3fn casts with the reference's power-of-two block-32 scale (quant.rs:190-214), quantisation of x
    in front of gate/up and of the SwiGLU output in front of down, where the reference's device chain quantises
    (kernels.rs:97-108,586-598).  Agreement to 1e-6 of the output's range; and statements that quantise differently
    (block 128, an unrounded scale, x only, the SwiGLU output only, one term where two are meant) are told apart."""
    inp = synth.make_inputs(cfg, seed=seed)
    # e4m3 is a floating-point format: under a power-of-two scale a value keeps its three mantissa bits whatever
    # block its scale was taken from, until it falls below the format's range (2^-15 of the block maximum).  So the
    # block size only shows when neighbouring blocks differ by more than that, and then only if the small blocks
    # still matter to the result.  Every other block of 32 is therefore made 2^-16 times smaller, in x and (through
    # the up projection's scales) in the SwiGLU output, and the weights that multiply those blocks 2^16 times
    # larger: the f32 result is of the same kind as before, a quantiser over 32 values still sees each block at its
    # own magnitude, and one over 128 flushes half of the blocks.
    H, I, Is = cfg.hidden, cfg.inter, cfg.shared_inter
    odd = lambda nblk: (np.arange(nblk) % 2) * 16
    inp.x = (inp.x * np.repeat(2.0 ** -odd(H // 32), 32)).astype(np.float32)
    for name in ("gate_s", "up_s", "sh_gate_s", "sh_up_s"):          # [.., rows, H/32]: columns of the small x blocks
        setattr(inp, name, (getattr(inp, name) + odd(H // 32)[None, None, :]).astype(np.uint8))
    for name, rows in (("up_s", I), ("sh_up_s", Is)):                # rows of the up projection -> small act blocks
        setattr(inp, name, (getattr(inp, name) - np.repeat(odd(rows // 32), 32)[None, :, None]).astype(np.uint8))
    for name, rows in (("down_s", I), ("sh_down_s", Is)):            # [.., H, I/32]: columns of the small act blocks
        setattr(inp, name, (getattr(inp, name) + odd(rows // 32)[None, None, :]).astype(np.uint8))
    f32 = oracle.moe_ffn_mxfp4(inp, act_mode=0)
    ids, probs = f32["ids"].astype(int), f32["probs"].astype(np.float64)
    q1, q2 = refmath.qdq_e4m3, refmath.qdq_e4m3_x2
    q2_128 = lambda a: q1(a, block=128) + q1(np.asarray(a, np.float32) - q1(a, block=128).astype(np.float32), block=128)
    got1 = oracle.moe_ffn_mxfp4(inp, act_mode=1)
    got2 = oracle.moe_ffn_mxfp4(inp, act_mode=2)
    for got in (got1, got2):       # routing sees the unquantised x
        assert np.array_equal(got["ids"], f32["ids"]) and np.array_equal(got["probs"], f32["probs"])
    ref1 = refmath.moe_layer(inp, ids, probs, quant_x=q1, quant_act=q1)[0]
    ref2 = refmath.moe_layer(inp, ids, probs, quant_x=q2, quant_act=q2)[0]
    assert refmath.max_abs_rel(got1["out"], ref1) < 1e-6
    # the second term quantises a residual sixteen times smaller than the value, so the last-bit differences between
    # this float64 SwiGLU and the oracle's f32 one move a rounding decision now and then: one e4m3 step of a
    # residual, 2^-8 of one activation
    assert refmath.max_abs_rel(got2["out"], ref2) < 1e-5
    wrong = {
        "block 128": dict(quant_x=lambda a: refmath.qdq_e4m3(a, block=128), quant_act=lambda a: refmath.qdq_e4m3(a, block=128)),
        "scale not a power of two": dict(quant_x=lambda a: refmath.qdq_e4m3(a, pow2_scale=False),
                                         quant_act=lambda a: refmath.qdq_e4m3(a, pow2_scale=False)),
        "x only": dict(quant_x=q1, quant_act=None),
        "SwiGLU output only": dict(quant_x=None, quant_act=q1),
        "two terms": dict(quant_x=q2, quant_act=q2),
    }
    for name, kw in wrong.items():
        assert refmath.max_abs_rel(got1["out"], refmath.moe_layer(inp, ids, probs, **kw)[0]) > 1e-3, name
    for name, kw in {"one term": dict(quant_x=q1, quant_act=q1), "second term on x only": dict(quant_x=q2, quant_act=q1),
                     "second term on the SwiGLU output only": dict(quant_x=q1, quant_act=q2),
                     "block 128": dict(quant_x=q2_128, quant_act=q2_128), "no quantisation": dict()}.items():
        assert refmath.max_abs_rel(got2["out"], refmath.moe_layer(inp, ids, probs, **kw)[0]) > 2e-4, name
    # distances to the f32 golden (CpuBackend proper): one e4m3 term is a few percent, two are bf16-class
    d1, d2 = refmath.max_abs_rel(got1["out"], f32["out"]), refmath.max_abs_rel(got2["out"], f32["out"])
    assert 5e-3 < d1 < 8e-2 and d2 < 5e-3 and d2 < d1 / 8, (d1, d2)


def test_two_term_quantiser_is_the_quantiser_twice(oracle):
    """fo_act_quant_fp8_x2 = act_quant_fp8 of x, then of x - dq1 (f32), bit for bit; and the two terms together
    represent x far better than one (residual below 2^-7 of the block maximum)."""
    rng = np.random.default_rng(4)
    x = np.concatenate([rng.normal(0, 1, 4096), rng.normal(0, 1e-3, 512), rng.uniform(-500, 500, 512),
                        np.zeros(64), [448.0, -448.0, 7.6 / 512, 1e-30] * 8]).astype(np.float32)
    q1, s1, q2, s2 = oracle.act_quant_fp8_x2(x)
    a1, b1 = oracle.act_quant_fp8(x, 32, True)
    dq1 = np.array([oracle.e4m3_decode(int(b)) for b in a1], np.float32) * np.repeat(b1, 32)
    a2, b2 = oracle.act_quant_fp8(x - dq1, 32, True)
    assert np.array_equal(q1, a1) and np.array_equal(s1, b1) and np.array_equal(q2, a2) and np.array_equal(s2, b2)
    dq2 = np.array([oracle.e4m3_decode(int(b)) for b in q2], np.float32) * np.repeat(s2, 32)
    assert np.allclose(refmath.qdq_e4m3_x2(x), (dq1 + dq2).astype(np.float64), rtol=0, atol=0)
    amax = np.repeat(np.abs(x.reshape(-1, 32)).max(axis=1), 32)
    assert (np.abs(x - (dq1 + dq2)) <= amax * 2.0 ** -7 + 1e-37).all()
    assert np.abs(x - dq1).max() >= 16 * np.abs(x - (dq1 + dq2)).max()   # four more bits at the least


def test_golden_c0(oracle):
    path = os.path.join(os.path.dirname(__file__), "golden", "c0_layer.npz")
    g = np.load(path)
    inp = synth.make_inputs(synth.CONFIGS["c0"], seed=0)
    got = oracle.moe_ffn_mxfp4(inp)
    assert np.array_equal(got["ids"].astype(np.int32), g["ids"])
    assert np.array_equal(got["probs"], g["probs"])
    assert np.array_equal(got["logits"], g["logits"])
    assert np.array_equal(got["out"], g["out_f32"])
    assert np.array_equal(oracle.moe_ffn_mxfp4(inp, act_mode=1)["out"], g["out_fp8act"])
    assert np.array_equal(oracle.moe_ffn_mxfp4(inp, act_mode=2)["out"], g["out_fp8x2"])
    t = oracle.moe_permute(g["ids"], inp.cfg.n_experts)
    for k in ("counts", "starts", "perm_map", "gather_src"):
        assert np.array_equal(t[k], g[k])
