"""The oracle's CpuBackend ops and permutation against the reference's own golden tests
(crates/ferrite-kernel/tests/golden.rs, gpu_smoke.rs:139-155, dsv41/chain_dev.rs:25042-25090,
dsv41/ops.rs:1079-1105) plus closed forms and brute force."""
import itertools
import math

import numpy as np
import pytest


def sigmoid32(v):
    v = np.float32(v)
    return np.float32(1.0) / (np.float32(1.0) + np.float32(math.exp(-float(v))))


def test_matmul_matches_manual(oracle):  # golden.rs:14-27
    x = np.array([[1, 2], [3, 4]], np.float32)
    w = np.array([[5, 6], [7, 8]], np.float32)
    assert oracle.matmul(x, w).tolist() == [[17, 23], [39, 53]]
    assert oracle.matmul(x, w, np.array([0.5, -0.5], np.float32)).tolist() == [[17.5, 22.5], [39.5, 52.5]]
    with pytest.raises(oracle.OracleError):
        oracle.matmul(x, np.zeros((2, 3), np.float32))


def test_matmul_is_sequential_f32_chain(oracle):
    """Bit-for-bit equal to s=0; s = fl(s + fl(x*w)) in index order; the 8-row interleave in the
    oracle must not change any chain (rows 0..18 exercise both the blocked and the tail path)."""
    rng = np.random.default_rng(0)
    x = rng.normal(0, 1, (3, 301)).astype(np.float32)
    w = rng.normal(0, 1, (19, 301)).astype(np.float32)
    got = oracle.matmul(x, w)
    for i in range(3):
        for j in range(19):
            s = np.float32(0)
            for l in range(301):
                s = np.float32(s + np.float32(x[i, l] * w[j, l]))
            assert got[i, j] == s
    # and it is NOT the fused-multiply-add chain on at least one element (contraction is off)
    diff = 0
    for j in range(19):
        s = 0.0
        sf = np.float32(0)
        for l in range(301):
            sf = np.float32(float(sf) + float(x[0, l]) * float(w[j, l]))  # fma-like: one rounding
        diff += int(sf != got[0, j])
    assert diff > 0


def test_swiglu_clamps(oracle):  # golden.rs:44-55
    out = oracle.swiglu_limited(np.array([[2., 20., 3., 1.]], np.float32), 10.0)
    silu2 = 2.0 / (1.0 + math.exp(-2.0))
    assert abs(out[0, 0] - silu2 * 3.0) < 1e-6
    assert abs(out[0, 1] - 10.0 / (1.0 + math.exp(-10.0))) < 1e-6


def test_swiglu_up_clamps_both_sides(oracle):  # dsv41 ops.rs:1100-1105: silu(10) * -10
    out = oracle.swiglu_limited(np.array([[100., -100.]], np.float32), 10.0)
    assert abs(out[0, 0] - (10.0 / (1.0 + math.exp(-10.0))) * -10.0) < 1e-4
    out = oracle.swiglu_limited(np.array([[-100., 100.]], np.float32), 10.0)   # gate is not clamped below
    assert abs(out[0, 0] - (-100.0 / (1.0 + math.exp(100.0))) * 10.0) < 1e-30


def test_moe_route_noaux_tc(oracle):  # golden.rs:189-210
    probs, ids = oracle.moe_route(np.array([[1.0, 2.0, 0.5]]), np.array([0.0, 0.0, 0.5]), 2, 1.0)
    assert ids.tolist() == [[2.0, 1.0]]
    s1, s2 = sigmoid32(2.0), sigmoid32(0.5)
    assert abs(probs[0, 0] - s2 / (s1 + s2)) < 1e-5
    assert abs(probs[0, 1] - s1 / (s1 + s2)) < 1e-5


def test_moe_route_bias_selects_but_does_not_scale(oracle):  # dsv41 ops.rs:1079-1087
    probs, ids = oracle.moe_route(np.array([[1.0, 1.0]]), np.array([0.0, 10.0]), 1, 1.0)
    assert ids[0, 0] == 1.0
    s = float(sigmoid32(1.0))
    assert abs(probs[0, 0] - s / (s + np.finfo(np.float32).eps)) < 1e-6


def ramp_fixture():
    n, e, topk = 2, 288, 8
    logits = (np.arange(n * e, dtype=np.float32) * np.float32(0.017) - np.float32(2.0)).reshape(n, e)
    bias = ((np.arange(e) % 11).astype(np.float32) * np.float32(0.01))
    return logits, bias, topk


def test_moe_route_ramp_fixture_closed_form(oracle):  # gpu_smoke.rs:139-155 inputs
    logits, bias, topk = ramp_fixture()
    probs, ids = oracle.moe_route(logits, bias, topk, 2.5)
    for r in range(2):
        sig = 1.0 / (1.0 + np.exp(-logits[r].astype(np.float64)))
        choice = sig + bias
        order = sorted(range(288), key=lambda j: (-choice[j], j))[:topk]
        assert ids[r].astype(int).tolist() == order
        want = sig[order] / sig[order].sum() * 2.5
        assert np.allclose(probs[r], want, atol=1e-5)
        assert len(set(order)) == topk
        assert abs(probs[r].sum() - 2.5) < 1e-4


def test_moe_route_ties_go_to_lower_index_and_order_is_by_choice(oracle):  # cpu.rs:560
    logits = np.zeros((1, 8), np.float32)
    probs, ids = oracle.moe_route(logits, np.zeros(8, np.float32), 3, 1.0)
    assert ids.tolist() == [[0.0, 1.0, 2.0]]
    bias = np.array([0, 0.25, 0, 0.25, 0.5, 0, 0, 0], np.float32)
    _, ids = oracle.moe_route(logits, bias, 4, 1.0)
    assert ids.tolist() == [[4.0, 1.0, 3.0, 0.0]]


def test_moe_route_brute_force_small(oracle):
    rng = np.random.default_rng(2)
    for _ in range(50):
        e, k = int(rng.integers(2, 9)), 0
        k = int(rng.integers(1, e + 1))
        logits = rng.normal(0, 2, (1, e)).astype(np.float32)
        bias = rng.normal(0, 0.3, e).astype(np.float32)
        probs, ids = oracle.moe_route(logits, bias, k, 1.7)
        sig = np.array([sigmoid32(v) for v in logits[0]], np.float32)
        choice = (sig + bias).astype(np.float32)
        # the k chosen experts maximise the sum of choice scores over all k-subsets
        best = max(itertools.combinations(range(e), k), key=lambda c: sum(float(choice[j]) for j in c))
        assert sorted(ids[0].astype(int).tolist()) == sorted(best)
        ch = [float(choice[int(j)]) for j in ids[0]]
        assert ch == sorted(ch, reverse=True)
        s = np.float32(0)
        for j in ids[0].astype(int):
            s = np.float32(s + sig[j])
        want = [np.float32(np.float32(sig[j] / np.float32(s + np.finfo(np.float32).eps)) * np.float32(1.7))
                for j in ids[0].astype(int)]
        assert probs[0].tolist() == want


def test_moe_route_nan_is_an_error(oracle):  # the reference's partial_cmp().unwrap() panics
    with pytest.raises(oracle.OracleError):
        oracle.moe_route(np.array([[np.nan, 1.0]]), np.zeros(2), 1, 1.0)
    with pytest.raises(oracle.OracleError):
        oracle.moe_route(np.zeros((1, 4)), np.zeros(3), 1, 1.0)


# ---- group-limited routing: no reference counterpart (parity unpinned); pinned by reduction + brute force
def test_grouped_reduces_to_plain_router(oracle):
    rng = np.random.default_rng(4)
    logits = rng.normal(0, 1.5, (16, 32)).astype(np.float32)
    bias = rng.normal(0, 0.05, 32).astype(np.float32)
    p0, i0 = oracle.moe_route(logits, bias, 6, 2.5)
    for ng, tg in [(1, 1), (4, 4), (8, 8), (32, 32)]:
        p, i = oracle.moe_route(logits, bias, 6, 2.5, ng, tg)
        assert np.array_equal(i, i0) and np.array_equal(p, p0)


def test_grouped_brute_force_c0_shape(oracle):
    """E=16, 4 groups keep 2, top-4: enumerate all C(4,2) group subsets."""
    rng = np.random.default_rng(6)
    logits = rng.normal(0, 1.5, (64, 16)).astype(np.float32)
    bias = rng.normal(0, 0.05, 16).astype(np.float32)
    probs, ids = oracle.moe_route(logits, bias, 4, 2.5, 4, 2)
    for r in range(64):
        sig = np.array([sigmoid32(v) for v in logits[r]], np.float32)
        choice = (sig + bias).astype(np.float32)
        gscore = []
        for g in range(4):
            top2 = sorted(choice[g * 4:(g + 1) * 4].tolist(), reverse=True)[:2]
            gscore.append(float(np.float32(np.float32(top2[0]) + np.float32(top2[1]))))
        best = max(itertools.combinations(range(4), 2), key=lambda c: (gscore[c[0]] + gscore[c[1]]))
        kept = sorted(range(4), key=lambda g: (-gscore[g], g))[:2]
        assert sorted(kept) == sorted(best)
        cand = [j for j in range(16) if j // 4 in kept]
        want = sorted(cand, key=lambda j: (-float(choice[j]), j))[:4]
        assert ids[r].astype(int).tolist() == want
        assert all(int(j) // 4 in kept for j in ids[r])


def test_grouped_rejects_bad_shapes(oracle):
    z = np.zeros((1, 16), np.float32)
    with pytest.raises(oracle.OracleError):
        oracle.moe_route(z, np.zeros(16), 4, 1.0, 3, 2)      # E % n_group
    with pytest.raises(oracle.OracleError):
        oracle.moe_route(z, np.zeros(16), 9, 1.0, 4, 2)      # topk > kept experts


# ---- permutation
def test_moe_align_host_groups_stably_and_zero_fills(oracle):  # chain_dev.rs:25042-25061
    BM, CAP = 8, 16
    order, counts, eid, nseg = oracle.moe_align_host([5, 1, 5, 1, 5, 2, 9, 1, 9], 3, CAP, BM)
    assert nseg == 4
    assert eid[:4].tolist() == [1, 2, 5, 9]
    assert counts[:4].tolist() == [3, 1, 3, 2]
    assert order[0:3].tolist() == [1, 3, 7]
    assert order[BM:BM + 1].tolist() == [5]
    assert order[2 * BM:2 * BM + 3].tolist() == [0, 2, 4]
    assert order[3 * BM:3 * BM + 2].tolist() == [6, 8]
    assert order[3] == -1 and np.all(order[nseg * BM:] == -1) and np.all(counts[nseg:] == 0)


def test_moe_align_host_declines_out_of_contract(oracle):  # chain_dev.rs:25077-25090
    assert oracle.moe_align_host([], 6, 16, 8) is None
    assert oracle.moe_align_host([0, 1, 2], 0, 16, 8) is None
    assert oracle.moe_align_host([0, -1, 2], 3, 16, 8) is None
    assert oracle.moe_align_host(list(range(17)), 1, 16, 8) is None
    assert oracle.moe_align_host([7] * 9, 1, 16, 8) is None


def test_moe_permute_reference_vector(oracle):  # same routing table, dsv41_route.cu:194-225 tables
    ids = np.array([[5, 1, 5], [1, 5, 2], [9, 1, 9]], np.int32)
    t = oracle.moe_permute(ids, 12)
    assert t["counts"].tolist() == [0, 3, 1, 0, 0, 3, 0, 0, 0, 2, 0, 0]
    assert t["gather_src"].tolist() == [1, 3, 7, 5, 0, 2, 4, 6, 8]
    assert t["active"][:t["n_active"]].tolist() == [1, 2, 5, 9] and t["n_active"] == 4
    assert t["starts"].tolist() == [0, 0, 3, 4, 4, 4, 7, 7, 7, 7, 9, 9, 9]
    assert t["perm_map"].tolist() == [4, 0, 5, 1, 6, 3, 7, 2, 8]


def test_moe_permute_is_stable_sort_and_invariants(oracle):
    rng = np.random.default_rng(8)
    for n, k, e in [(1, 1, 1), (7, 3, 5), (64, 8, 128), (300, 8, 256)]:
        ids = np.stack([rng.permutation(e)[:k] if k <= e else rng.integers(0, e, k) for _ in range(n)]).astype(np.int32)
        t = oracle.moe_permute(ids, e)
        flat = ids.ravel()
        want = np.argsort(flat, kind="stable")
        assert np.array_equal(t["gather_src"], want)
        assert np.array_equal(t["perm_map"][t["gather_src"]], np.arange(n * k))
        assert np.array_equal(t["counts"], np.bincount(flat, minlength=e))
        assert np.array_equal(t["starts"], np.concatenate([[0], np.cumsum(t["counts"])]))
        assert t["counts"].sum() == n * k


def test_moe_permute_out_of_range_ids_drop_out(oracle):  # dsv41_route.cu:253-261,300-303
    ids = np.array([[0, 7], [-1, 0]], np.int32)
    t = oracle.moe_permute(ids, 4)
    assert t["perm_map"].tolist() == [0, -1, -1, 1]
    assert t["gather_src"].tolist() == [0, 3, -1, -1]
    assert t["starts"][-1] == 2


# ---- the steps before and after the layer: rmsnorm (cpu.rs:124-143), hc_post (cpu.rs:788-807) ----
def _rmsnorm_f32_steps(x, w, eps):
    """The reference's evaluation order, one rounded f32 operation at a time."""
    f = np.float32
    out = np.empty_like(x)
    for i, row in enumerate(x):
        ss = f(0.0)
        for v in row:
            ss = f(ss + f(v * v))
        ss = f(ss / f(len(row)))
        inv = f(f(1.0) / np.sqrt(f(ss + f(eps)), dtype=np.float32))
        for j, v in enumerate(row):
            out[i, j] = f(f(v * inv) * w[j])
    return out


def test_rmsnorm_manual(oracle):  # golden.rs:30-42
    x = np.array([[1., 2., 3., 4.]], np.float32)
    out = oracle.rmsnorm(x, np.ones(4, np.float32), 1e-6)
    inv = np.float32(1.0) / np.sqrt(np.float32((1 + 4 + 9 + 16) / 4) + np.float32(1e-6), dtype=np.float32)
    assert np.abs(out[0] - x[0] * inv).max() < 1e-5           # the reference test's own bar
    assert np.array_equal(out, _rmsnorm_f32_steps(x, np.ones(4, np.float32), 1e-6))


def test_rmsnorm_is_the_sequential_f32_evaluation(oracle):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((3, 517)) * np.array([[1e-3], [1.0], [300.0]])).astype(np.float32)
    w = rng.uniform(0.5, 1.5, 517).astype(np.float32)
    got = oracle.rmsnorm(x, w, 1e-5)
    assert np.array_equal(got, _rmsnorm_f32_steps(x, w, 1e-5))
    # a row on which the left-to-right f32 sum differs from a pairwise or float64 sum: 1 followed by many 2^-13
    # (each square 2^-26 is below half an ulp of 1 and is dropped one at a time, but not when summed first)
    row = np.full((1, 4097), 2.0 ** -13, np.float32)
    row[0, 0] = 1.0
    seq = oracle.rmsnorm(row, np.ones(4097, np.float32), 0.0)
    ss64 = np.float32(np.sum(row.astype(np.float64) ** 2) / 4097)
    other = row * (np.float32(1.0) / np.sqrt(ss64, dtype=np.float32))
    assert np.array_equal(seq, _rmsnorm_f32_steps(row, np.ones(4097, np.float32), 0.0))
    assert not np.array_equal(seq, other)
    # unit mean square once eps is negligible against the row's mean square (rows 1 and 2)
    ms = np.mean(got[1:].astype(np.float64) ** 2 / w.astype(np.float64) ** 2, axis=1)
    assert np.abs(ms - 1.0).max() < 1e-3
    with pytest.raises(oracle.OracleError):
        oracle.rmsnorm(x, w[:-1], 1e-5)


def _hc_post_f32_steps(x, res, post, comb):
    f = np.float32
    s, nh, h = res.shape
    out = np.empty_like(res)
    for t in range(s):
        for i in range(nh):
            acc = (post[t, i] * x[t]).astype(f)
            for k in range(nh):
                acc = (acc + (comb[t, k, i] * res[t, k]).astype(f)).astype(f)
            out[t, i] = acc
    return out


def test_hc_post_reference_fixture_and_special_cases(oracle):
    # inputs of gpu_smoke.rs:337-343 (s=2, n=4, h=64); post/comb there come from hc_pre, any values pin the formula
    s, nh, h = 2, 4, 64
    x = ((np.arange(s * h) * 7 % 31) * 0.03).astype(np.float32).reshape(s, h)
    res = ((np.arange(s * nh * h) * 13 % 47) * 0.02 - 0.5).astype(np.float32).reshape(s, nh, h)
    rng = np.random.default_rng(9)
    post = rng.uniform(0, 2, (s, nh)).astype(np.float32)          # sigmoid range of hc_pre (mhc.rs:252-255)
    comb = rng.uniform(0, 1, (s, nh, nh)).astype(np.float32)
    got = oracle.hc_post(x, res, post, comb)
    assert got.shape == (s, nh, h)
    assert np.array_equal(got, _hc_post_f32_steps(x, res, post, comb))
    # the mix is comb[t, k, i] (column i), not comb[t, i, k]: a non-symmetric comb tells them apart
    assert not np.array_equal(got, _hc_post_f32_steps(x, res, post, comb.transpose(0, 2, 1).copy()))
    # identity mix and unit post: out[t, i] = x[t] + residual[t, i], exactly
    eye = np.broadcast_to(np.eye(nh, dtype=np.float32), (s, nh, nh)).copy()
    one = np.ones((s, nh), np.float32)
    assert np.array_equal(oracle.hc_post(x, res, one, eye), x[:, None, :] + res)
    # zero mix: out = post * x
    assert np.array_equal(oracle.hc_post(x, res, post, np.zeros_like(comb)), post[:, :, None] * x[:, None, :])
    with pytest.raises(oracle.OracleError):
        oracle.hc_post(x, res, post[:, :2], comb)


def test_route_nan_scores_device_policy(oracle):
    """CpuBackend panics on a NaN score (cpu.rs:560: partial_cmp().unwrap()); the reference's device router never
    selects one and marks slots it cannot fill with id -1, weight 0 (kernels/cuda/ferrite_kernels.cu:1233-1270).
    The oracle states both; the second is pinned by its special cases: without NaN it is the first, a NaN expert
    is as good as absent (the remaining experts route as if it scored -inf), all-NaN gives all -1."""
    rng = np.random.default_rng(5)
    logits = rng.normal(0, 1.5, (6, 32)).astype(np.float32)
    bias = rng.normal(0, 0.01, 32).astype(np.float32)
    for ng, tg in ((1, 1), (4, 2)):
        p0, i0 = oracle.moe_route(logits, bias, 4, 2.5, ng, tg)
        p1, i1 = oracle.moe_route(logits, bias, 4, 2.5, ng, tg, nan_policy=1)
        assert np.array_equal(p0, p1) and np.array_equal(i0, i1)
    bad = logits.copy()
    bad[0, 3] = np.nan
    bad[1, :] = np.nan
    bad[2, :30] = np.nan          # two finite scores for four slots
    with pytest.raises(oracle.OracleError):
        oracle.moe_route(bad, bias, 4, 2.5)
    p, i = oracle.moe_route(bad, bias, 4, 2.5, nan_policy=1)
    # row 0: expert 3 absent == the same row with a hugely negative logit there (sigmoid 0, bias cannot lift it)
    sub = logits[:1].copy()
    sub[0, 3] = -1e30
    big_neg_bias = bias.copy()
    big_neg_bias[3] = -10.0
    ps, is_ = oracle.moe_route(sub, big_neg_bias, 4, 2.5)
    assert np.array_equal(i[0], is_[0]) and np.array_equal(p[0], ps[0]) and 3 not in i[0]
    assert i[1].tolist() == [-1, -1, -1, -1] and p[1].tolist() == [0, 0, 0, 0]
    assert sorted(i[2, :2].tolist()) == [30, 31] and i[2, 2:].tolist() == [-1, -1] and p[2, 2:].tolist() == [0, 0]
    assert abs(p[2, :2].sum() - 2.5) < 1e-5
    assert np.array_equal(i[3:], oracle.moe_route(logits, bias, 4, 2.5)[1][3:])
    # grouped: a group whose experts are all NaN ranks last and is dropped when enough other groups exist
    g = logits.copy()
    g[:, 8:16] = np.nan
    pg, ig = oracle.moe_route(g, bias, 4, 2.5, 4, 2, nan_policy=1)
    assert ((ig < 8) | (ig >= 16)).all() and (ig >= 0).all()
