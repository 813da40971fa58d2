"""GPU parity of the op-level entry points against the CPU oracle, through the C ABI.
Integer/byte results and everything routing depends on are compared bit for bit."""
import numpy as np
import pytest
import torch

from ferrite_amd import synth
from ferrite_amd.backend import InvalidArg, ShapeMismatch

pytestmark = pytest.mark.gpu


def dev(hip, a, dtype=None):
    return hip.upload(np.asarray(a), dtype)


def host(hip, t):
    hip.sync()
    return t.cpu().numpy()


# ---- matmul: the reference's sequential-k chain, bit for bit ----
def test_matmul_matches_manual(hip):  # golden.rs:14-27
    x, w = dev(hip, np.array([[1, 2], [3, 4]], np.float32)), dev(hip, np.array([[5, 6], [7, 8]], np.float32))
    out = torch.zeros(2, 2, device=hip.device)
    hip.matmul(x, w, None, out)
    assert host(hip, out).tolist() == [[17, 23], [39, 53]]
    hip.matmul(x, w, dev(hip, np.array([0.5, -0.5], np.float32)), out)
    assert host(hip, out).tolist() == [[17.5, 22.5], [39.5, 52.5]]


@pytest.mark.parametrize("n,k,o", [(5, 300, 70), (32, 4096, 128), (3, 37, 5), (1, 64, 1), (130, 256, 16), (7, 7168, 256)])
def test_matmul_bit_exact_vs_oracle(hip, oracle, n, k, o):
    rng = np.random.default_rng(n * 1000 + k)
    x = rng.normal(0, 1, (n, k)).astype(np.float32)
    w = rng.normal(0, 0.02, (o, k)).astype(np.float32)
    b = rng.normal(0, 1, o).astype(np.float32)
    out = torch.empty(n, o, device=hip.device)
    hip.matmul(dev(hip, x), dev(hip, w), None, out)
    assert np.array_equal(host(hip, out), oracle.matmul(x, w))
    hip.matmul(dev(hip, x), dev(hip, w), dev(hip, b), out)
    assert np.array_equal(host(hip, out), oracle.matmul(x, w, b))


def test_matmul_shape_errors(hip):
    z = lambda *s: torch.zeros(*s, device=hip.device)
    with pytest.raises(ShapeMismatch):
        hip.matmul(z(2, 3), z(2, 4), None, z(2, 2))
    with pytest.raises(InvalidArg):
        hip.matmul(z(2, 3), z(4, 3), None, z(2, 2))


# ---- swiglu ----
def test_swiglu_bit_exact_vs_oracle(hip, oracle):  # golden.rs:44-55 values included
    rng = np.random.default_rng(1)
    gu = rng.normal(0, 4, (17, 2 * 96)).astype(np.float32)
    gu[0, :4] = [2., 20., -200., 95.]
    gu[0, 96:100] = [3., 1., 50., -50.]
    out = torch.empty(17, 96, device=hip.device)
    hip.swiglu_limited(dev(hip, gu), 10.0, out)
    assert np.array_equal(host(hip, out), oracle.swiglu_limited(gu, 10.0))
    with pytest.raises(InvalidArg):
        hip.swiglu_limited(dev(hip, gu[:, :191]), 10.0, out)


# ---- routing ----
def route(hip, logits, bias, k, scale, ng=1, tg=1):
    n = logits.shape[0]
    probs = torch.empty(n, k, device=hip.device)
    ids = torch.empty(n, k, device=hip.device)
    ids32 = torch.empty(n, k, dtype=torch.int32, device=hip.device)
    hip.moe_route(dev(hip, logits.astype(np.float32)), dev(hip, bias.astype(np.float32)), k, scale, probs, ids, ng, tg, ids32)
    p, i, i32 = host(hip, probs), host(hip, ids), host(hip, ids32)
    assert np.array_equal(i.astype(np.int32), i32)
    return p, i


def test_moe_route_noaux_tc(hip):  # golden.rs:189-210
    p, i = route(hip, np.array([[1.0, 2.0, 0.5]]), np.array([0.0, 0.0, 0.5]), 2, 1.0)
    assert i.tolist() == [[2.0, 1.0]]
    s = lambda v: 1.0 / (1.0 + np.exp(-v))
    assert abs(p[0, 0] - s(0.5) / (s(2.0) + s(0.5))) < 1e-5 and abs(p[0, 1] - s(2.0) / (s(2.0) + s(0.5))) < 1e-5


def test_moe_route_ramp_fixture(hip, oracle):  # gpu_smoke.rs:139-155: ids exact, probs 1e-5 (here: exact)
    n, e, k = 2, 288, 8
    logits = (np.arange(n * e, dtype=np.float32) * np.float32(0.017) - np.float32(2.0)).reshape(n, e)
    bias = (np.arange(e) % 11).astype(np.float32) * np.float32(0.01)
    p, i = route(hip, logits, bias, k, 2.5)
    po, io = oracle.moe_route(logits, bias, k, 2.5)
    assert np.array_equal(i, io) and np.array_equal(p, po)


@pytest.mark.parametrize("n,e,k,ng,tg", [(8, 16, 4, 4, 2), (32, 128, 8, 8, 4), (33, 256, 8, 8, 4), (64, 128, 8, 1, 1),
                                         (5, 288, 8, 1, 1), (4, 64, 6, 4, 3), (16, 512, 32, 16, 8), (3, 8, 8, 1, 1)])
def test_moe_route_bit_exact_vs_oracle(hip, oracle, n, e, k, ng, tg):
    rng = np.random.default_rng(e + n)
    logits = rng.normal(0, 1.7, (n, e)).astype(np.float32)
    bias = rng.normal(0, 0.01, e).astype(np.float32)
    p, i = route(hip, logits, bias, k, 2.5, ng, tg)
    po, io = oracle.moe_route(logits, bias, k, 2.5, ng, tg)
    assert np.array_equal(i, io)
    assert np.array_equal(p, po)


def test_moe_route_ties_lower_index_first(hip, oracle):  # cpu.rs:560
    logits = np.zeros((2, 128), np.float32)
    bias = np.zeros(128, np.float32)
    bias[[5, 70, 9]] = 0.25
    for ng, tg in [(1, 1), (8, 4)]:
        p, i = route(hip, logits, bias, 8, 1.0, ng, tg)
        po, io = oracle.moe_route(logits, bias, 8, 1.0, ng, tg)
        assert np.array_equal(i, io) and np.array_equal(p, po)
    assert route(hip, logits, bias, 8, 1.0)[1][0].tolist() == [5, 9, 70, 0, 1, 2, 3, 4]


def test_moe_route_extreme_logits(hip, oracle):
    logits = np.array([[-200, -100, -88.5, -30, 0, 30, 88.5, 100, 200, 1e-30, -1e-30, 17.3, -17.3, 5, -5, 0.1]], np.float32)
    p, i = route(hip, logits, np.zeros(16, np.float32), 8, 2.5)
    po, io = oracle.moe_route(logits, np.zeros(16, np.float32), 8, 2.5)
    assert np.array_equal(i, io) and np.array_equal(p, po)


def test_moe_route_nan_scores(hip, oracle):
    """NaN logits: never selected; slots that no finite score can fill get id -1 and weight 0, as the reference's
    device router leaves them (kernels/cuda/ferrite_kernels.cu:1233-1270).  Bit-equal to the oracle's statement of
    that policy, grouped and ungrouped, and through the fused layer: such slots contribute nothing."""
    rng = np.random.default_rng(11)
    logits = rng.normal(0, 1.5, (8, 64)).astype(np.float32)
    bias = rng.normal(0, 0.01, 64).astype(np.float32)
    logits[0, 5] = np.nan
    logits[1, :] = np.nan
    logits[2, :61] = np.nan
    logits[3, 16:32] = np.nan
    logits[4, ::2] = np.nan
    for ng, tg in ((1, 1), (4, 2)):
        p, i = route(hip, logits, bias, 6, 2.5, ng, tg)
        po, io = oracle.moe_route(logits, bias, 6, 2.5, ng, tg, nan_policy=1)
        assert np.array_equal(i, io), (ng, tg)
        assert np.array_equal(p, po), (ng, tg)
    assert i[1].tolist() == [-1] * 6 and p[1].tolist() == [0.0] * 6


def test_layer_with_nan_activations_keeps_other_tokens_intact(hip, oracle):
    """A token whose activations are NaN routes nowhere (ids -1, no row in the permutation); every other token's row
    is bit-identical to a run without it, in both the fused-head and the separate-launch path."""
    from ferrite_amd import synth
    from ferrite_amd.backend import MODE_MFMA_FP8
    for n in (24, 300):
        cfg = synth.MoeConfig(n, 256, 16, 4, 128, 128, 4, 2)
        inp = synth.make_inputs(cfg, seed=n)
        layer = hip.load_moe_layer(inp)
        x = torch.from_numpy(inp.x).to(hip.device)
        out = torch.empty_like(x)
        hip.moe_layer_dev_mxfp4(layer, x, out, MODE_MFMA_FP8)
        hip.sync()
        clean = out.cpu().numpy()
        x[7, :] = float("nan")
        hip.moe_layer_dev_mxfp4(layer, x, out, MODE_MFMA_FP8)
        hip.sync()
        got = out.cpu().numpy()
        v = hip.workspace_view(layer, n, MODE_MFMA_FP8)
        assert v["ids"][7].cpu().tolist() == [-1] * 4
        assert v["perm_map"].view(n, 4)[7].cpu().tolist() == [-1] * 4
        keep = np.arange(n) != 7
        assert np.array_equal(got[keep], clean[keep])
        # (row 7 itself holds whatever the shared expert makes of the quantised row: the reference's e4m3 encoder
        # saturates non-finite values to +-448, quant.rs:98-124, so it need not be NaN)


def test_moe_route_shape_errors(hip):
    z = lambda *s: torch.zeros(*s, device=hip.device)
    with pytest.raises(InvalidArg):
        hip.moe_route(z(2, 8), z(7), 2, 1.0, z(2, 2), z(2, 2))
    with pytest.raises(InvalidArg):
        hip.moe_route(z(2, 8), z(8), 2, 1.0, z(2, 3), z(2, 2))
    with pytest.raises(InvalidArg):
        hip.moe_route(z(2, 8), z(8), 2, 1.0, z(2, 2), z(2, 2), 3, 2)   # E % n_group


# ---- permutation ----
def permute(hip, ids, e):
    t = hip.moe_permute(dev(hip, ids.astype(np.int32)), e)
    hip.sync()
    return {k: v.cpu().numpy() for k, v in t.items()}


def test_moe_permute_reference_vector(hip, oracle):  # chain_dev.rs:25042-25061 routing table, as it stands there
    """The reference's vector lists an expert twice inside a token (5,1,5 and 9,1,9); its order is
    [1,3,7] [5] [0,2,4] [6,8] for experts 1, 2, 5, 9 with counts 3, 1, 3, 2."""
    ids = np.array([[5, 1, 5], [1, 5, 2], [9, 1, 9]])
    t = permute(hip, ids, 12)
    assert t["gather_src"].tolist() == [1, 3, 7, 5, 0, 2, 4, 6, 8]
    assert t["counts"].tolist() == [0, 3, 1, 0, 0, 3, 0, 0, 0, 2, 0, 0]
    assert t["active"][:4].tolist() == [1, 2, 5, 9] and int(t["n_active"][0]) == 4
    o = oracle.moe_permute(ids, 12)
    for key in ("counts", "starts", "perm_map", "gather_src", "active"):
        assert np.array_equal(t[key], o[key]), key
    t = permute(hip, np.array([[5, 1, 7], [1, 5, 2], [9, 1, 3]]), 12)
    assert t["gather_src"].tolist() == [1, 3, 7, 5, 8, 0, 4, 2, 6]
    assert t["counts"].tolist() == [0, 3, 1, 1, 0, 2, 0, 1, 0, 1, 0, 0]


@pytest.mark.parametrize("n,k,e", [(40, 6, 5), (700, 8, 16), (3000, 4, 3)])
def test_moe_permute_repeated_experts_in_a_token(hip, oracle, n, k, e):
    """ids drawn with replacement: many tokens repeat an expert; also beyond the single-block path."""
    rng = np.random.default_rng(n)
    ids = rng.integers(0, e, (n, k)).astype(np.int32)
    t = permute(hip, ids, e)
    o = oracle.moe_permute(ids, e)
    for key in ("counts", "starts", "perm_map", "gather_src", "active"):
        assert np.array_equal(t[key], o[key]), key
    assert np.array_equal(t["gather_src"], np.argsort(ids.ravel(), kind="stable"))


@pytest.mark.parametrize("n,k,e", [(1, 1, 1), (7, 3, 5), (32, 8, 128), (192, 8, 128), (1000, 8, 256), (1024, 8, 128),
                                   (1025, 8, 128), (4096, 8, 128), (8192, 8, 256), (3000, 4, 16)])
def test_moe_permute_memcmp_vs_oracle(hip, oracle, n, k, e):
    rng = np.random.default_rng(n + e)
    pop = rng.dirichlet(np.full(e, 0.3))  # skewed expert popularity
    ids = np.stack([rng.choice(e, size=k, replace=False, p=pop) for _ in range(n)]).astype(np.int32)
    t = permute(hip, ids, e)
    o = oracle.moe_permute(ids, e)
    for key in ("counts", "starts", "perm_map", "gather_src", "active"):
        assert np.array_equal(t[key], o[key]), key
    assert int(t["n_active"][0]) == o["n_active"]
    assert np.array_equal(t["gather_src"], np.argsort(ids.ravel(), kind="stable"))


def test_moe_permute_out_of_range_ids_drop_out(hip, oracle):  # dsv41_route.cu:253-261,300-303
    ids = np.array([[0, 7], [-1, 0], [2, 1]], np.int32)
    t = permute(hip, ids, 4)
    o = oracle.moe_permute(ids, 4)
    for key in ("counts", "starts", "perm_map", "gather_src"):
        assert np.array_equal(t[key], o[key]), key


# ---- formats ----
def test_mxfp4_dequant_bit_exact(hip, oracle):
    rng = np.random.default_rng(3)
    w = rng.integers(0, 256, (96, 128), dtype=np.uint8)
    s = rng.integers(100, 140, (96, 8), dtype=np.uint8)
    got = host(hip, hip.mxfp4_dequant(dev(hip, w), dev(hip, s)))
    assert np.array_equal(got.view(np.uint32), oracle.dequant_fp4_row32(w, s).view(np.uint32))


def test_mxfp4_dequant_all_codes_and_layout(hip):  # quant.rs:459-478 nibble order, every code
    w = np.zeros((1, 16), np.uint8)
    w[0, 0] = 0b1001_0111                       # element 0 = code 7 (6.0), element 1 = code 9 (-0.5)
    w[0, 8:16] = (np.arange(0, 16, 2) | (np.arange(1, 16, 2) << 4)).astype(np.uint8)
    got = host(hip, hip.mxfp4_dequant(dev(hip, w), dev(hip, np.array([[128]], np.uint8))))[0]
    assert got[0] == 12.0 and got[1] == -1.0
    assert got[16:].tolist() == [0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_act_quant_bit_exact_vs_oracle(hip, oracle, dtype):
    rng = np.random.default_rng(4)
    x = (rng.normal(0, 1, (64, 256)) * np.repeat(10.0 ** rng.uniform(-4, 4, (64, 8)), 32, axis=1)).astype(np.float32)
    x[3, 32:64] = 0.0
    x[5, 0:32] = np.linspace(7.3 / 512, 8.1 / 512, 32) * 1.0   # the subnormal clamp rule after scaling by 2^0.. region
    x[5, 0] = 448.0
    xt = torch.from_numpy(x).to(dtype)
    xr = xt.to(torch.float32).numpy()
    q, s = hip.act_quant_fp8(xt.to(hip.device))
    qo, so = oracle.act_quant_fp8(xr, 32, True)
    assert np.array_equal(host(hip, q).ravel(), qo)
    sbytes = host(hip, s).ravel()
    assert np.array_equal(np.exp2(sbytes.astype(np.float64) - 127), so.astype(np.float64))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_act_quant_two_terms_bit_exact_vs_oracle(hip, oracle, dtype):
    """Both terms of the two-term quantiser: codes and scales equal the oracle's, which is the reference's
    quantiser applied to x and then to what it leaves over."""
    rng = np.random.default_rng(6)
    x = (rng.normal(0, 1, (48, 512)) * np.repeat(10.0 ** rng.uniform(-4, 4, (48, 16)), 32, axis=1)).astype(np.float32)
    x[2, 64:96] = 0.0
    x[4, 0:32] = np.linspace(7.3 / 512, 8.1 / 512, 32)
    x[4, 0] = 448.0
    x[6, 32:64] = 2.0 ** -120          # scales at the smallest normal
    xt = torch.from_numpy(x).to(dtype)
    xr = xt.to(torch.float32).numpy()
    q1, s1, q2, s2 = (host(hip, t).ravel() for t in hip.act_quant_fp8_x2(xt.to(hip.device)))
    o1, t1, o2, t2 = oracle.act_quant_fp8_x2(xr)
    assert np.array_equal(q1, o1) and np.array_equal(q2, o2)
    assert np.array_equal(np.exp2(s1.astype(np.float64) - 127), t1.astype(np.float64))
    assert np.array_equal(np.exp2(s2.astype(np.float64) - 127), t2.astype(np.float64))
    # the first term is the one-term quantiser's output
    q, s = hip.act_quant_fp8(xt.to(hip.device))
    assert np.array_equal(host(hip, q).ravel(), q1) and np.array_equal(host(hip, s).ravel(), s1)


def test_pack_is_a_pure_permutation(hip, oracle):
    """dequant(packed) == dequant(checkpoint layout) for every matrix of several experts, bit for bit."""
    cfg = synth.MoeConfig(4, 256, 3, 2, 128, 256, 1, 1)
    inp = synth.make_inputs(cfg, seed=5)
    layer = hip.load_moe_layer(inp)
    for e in range(cfg.n_experts + 1):
        for which, (wn, sn) in enumerate([("gate", "gate"), ("up", "up"), ("down", "down")]):
            if e < cfg.n_experts:
                w, s = getattr(inp, f"{wn}_w")[e], getattr(inp, f"{sn}_s")[e]
            else:
                w, s = getattr(inp, f"sh_{wn}_w")[0], getattr(inp, f"sh_{sn}_s")[0]
            got = host(hip, hip.packed_dequant(layer, e, which))
            assert np.array_equal(got, oracle.dequant_fp4_row32(w, s)), (e, which)


# ---- the steps before and after the layer ----
@pytest.mark.parametrize("n,dim", [(1, 4), (11, 4096), (3, 517), (5, 7168), (2, 9000), (3, 520), (7, 1028), (1500, 256)])
def test_rmsnorm_bit_exact_vs_oracle(hip, oracle, n, dim):  # gpu_smoke.rs:56-70 shape [11, 4096] included
    rng = np.random.default_rng(n * 1000 + dim)
    x = (rng.standard_normal((n, dim)) * rng.uniform(1e-3, 30, (n, 1))).astype(np.float32)
    w = rng.uniform(0.5, 1.5, dim).astype(np.float32)
    if dim == 4:
        x[0] = [1., 2., 3., 4.]                       # golden.rs:30-42
    out = torch.empty(n, dim, device=hip.device)
    hip.rmsnorm(torch.from_numpy(x).to(hip.device), torch.from_numpy(w).to(hip.device), 1e-5, out)
    hip.sync()
    assert np.array_equal(out.cpu().numpy(), oracle.rmsnorm(x, w, 1e-5))


def test_rmsnorm_sequential_sum_and_errors(hip, oracle):
    from ferrite_amd.backend import InvalidArg
    row = np.full((1, 4097), 2.0 ** -13, np.float32)   # the left-to-right f32 sum drops every small square
    row[0, 0] = 1.0
    w = np.ones(4097, np.float32)
    out = torch.empty(1, 4097, device=hip.device)
    hip.rmsnorm(torch.from_numpy(row).to(hip.device), torch.from_numpy(w).to(hip.device), 0.0, out)
    hip.sync()
    assert np.array_equal(out.cpu().numpy(), oracle.rmsnorm(row, w, 0.0))
    with pytest.raises(InvalidArg):
        hip.rmsnorm(torch.zeros(2, 8, device=hip.device), torch.zeros(7, device=hip.device), 1e-5,
                    torch.zeros(2, 8, device=hip.device))


@pytest.mark.parametrize("s,nh,h", [(2, 4, 64), (32, 4, 4096), (5, 2, 12), (3, 8, 7168)])
def test_hc_post_bit_exact_vs_oracle(hip, oracle, s, nh, h):  # gpu_smoke.rs:308-348 shape (2, 4, 64) included
    rng = np.random.default_rng(s * 100 + nh)
    x = rng.standard_normal((s, h)).astype(np.float32)
    res = rng.standard_normal((s, nh, h)).astype(np.float32)
    post = rng.uniform(0, 2, (s, nh)).astype(np.float32)
    comb = rng.uniform(0, 1, (s, nh, nh)).astype(np.float32)
    if (s, nh, h) == (2, 4, 64):
        x = ((np.arange(s * h) * 7 % 31) * 0.03).astype(np.float32).reshape(s, h)
        res = ((np.arange(s * nh * h) * 13 % 47) * 0.02 - 0.5).astype(np.float32).reshape(s, nh, h)
    d = lambda a: torch.from_numpy(a).to(hip.device)
    out = hip.hc_post(d(x), d(res), d(post), d(comb))
    hip.sync()
    assert np.array_equal(out.cpu().numpy(), oracle.hc_post(x, res, post, comb))


def test_hc_post_shape_errors(hip):
    from ferrite_amd.backend import Declined, ShapeMismatch
    z = lambda *sh: torch.zeros(*sh, device=hip.device)
    with pytest.raises(ShapeMismatch):
        hip.hc_post(z(2, 8), z(2, 4, 8), z(2, 3), z(2, 4, 4))
    with pytest.raises(Declined):
        hip.hc_post(z(2, 8), z(2, 9, 8), z(2, 9), z(2, 9, 9))     # more than 8 flows
