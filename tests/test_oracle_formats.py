"""The oracle's format primitives against the reference's known-answer tests
(crates/ferrite-models/src/dsv41/quant.rs:336-501), exhaustive code sweeps and torch's e4m3 cast."""
import math

import numpy as np
import pytest
import torch

FP4 = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, 0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]


def test_fp4_table_matches_reference(oracle):  # quant.rs:336-347
    assert [oracle.e2m1_decode(c) for c in range(16)] == FP4
    assert oracle.e2m1_decode(0b0111) == 6.0
    assert oracle.e2m1_decode(0b1111) == -6.0
    assert oracle.e2m1_decode(0b1000) == 0.0
    assert oracle.e2m1_decode(0b1001) == -0.5


def test_fp4_roundtrip_all_codes(oracle):  # quant.rs:349-367
    for code in range(16):
        v = oracle.e2m1_decode(code)
        assert oracle.e2m1_decode(oracle.e2m1_encode(v)) == v
    assert oracle.e2m1_decode(oracle.e2m1_encode(0.2)) == 0.0
    assert oracle.e2m1_decode(oracle.e2m1_encode(0.3)) == 0.5
    assert oracle.e2m1_decode(oracle.e2m1_encode(-5.7)) == -6.0
    assert oracle.e2m1_decode(oracle.e2m1_encode(100.0)) == 6.0


def test_fp4_pack_layout_and_dequant_row32(oracle):  # quant.rs:369-380, 459-478
    packed = np.zeros((1, 16), np.uint8)
    packed[0, 0] = (0b0111 & 0xF) | ((0b1001 & 0xF) << 4)  # element 0 = 6.0 (low), element 1 = -0.5 (high)
    d = oracle.dequant_fp4_row32(packed, np.array([[127]], np.uint8))
    assert d[0, 0] == 6.0 and d[0, 1] == -0.5 and np.all(d[0, 2:] == 0)
    d2 = oracle.dequant_fp4_row32(packed, np.array([[128]], np.uint8))
    assert d2[0, 0] == 12.0


def test_e4m3_known_values(oracle):  # quant.rs:382-396
    assert oracle.e4m3_decode(0b0100_0000) == 2.0
    assert oracle.e4m3_decode(0b0100_0010) == 2.5
    assert oracle.e4m3_decode(0b1100_0000) == -2.0
    assert oracle.e4m3_decode(0b0100_1000) == 4.0
    assert oracle.e4m3_decode(0b0111_1110) == 448.0
    assert oracle.e4m3_decode(0) == 0.0
    assert oracle.e4m3_decode(1) == 1.0 / 512.0


def test_e4m3_roundtrip_saturating(oracle):  # quant.rs:398-411
    for v in [0.0, 1.0, 2.5, -2.5, 448.0, -448.0, 0.001953125, 1e9, -1e9]:
        dec = oracle.e4m3_decode(oracle.e4m3_encode(v))
        want = min(max(v, -448.0), 448.0)
        ulp = max(abs(want) * 2.0 ** -3, 1.0 / 512.0)
        assert abs(dec - want) <= ulp
    assert oracle.e4m3_encode(1e9) == 0b0111_1110
    assert oracle.e4m3_encode(-1e9) == 0b1111_1110
    assert oracle.e4m3_encode(float("inf")) == 0x7E and oracle.e4m3_encode(float("nan")) in (0x7E, 0xFE)


def test_e4m3_decode_all_bytes_vs_torch(oracle):
    """All 256 codes against torch.float8_e4m3fn (an independent library routine)."""
    b = torch.arange(256, dtype=torch.uint8)
    t = b.view(torch.float8_e4m3fn).to(torch.float32)
    for i in range(256):
        if i & 0x7F == 0x7F:
            continue  # e4m3fn NaN; the reference's decoder never sees it (encode saturates at 0x7E)
        assert oracle.e4m3_decode(i) == t[i].item(), i


def test_e4m3_encode_vs_torch_cast(oracle):
    """RNE + saturation: a dense sweep of finite values in [-448, 448] against torch's cast.

    One documented deviation: the reference clamps the subnormal mantissa to 7 (quant.rs:108-112), so
    |x| in [7.5/512, 8/512) encodes as 7/512 where IEEE-style RNE (torch) gives the smallest normal 8/512.
    The oracle follows the reference."""
    rng = np.random.default_rng(1)
    xs = np.concatenate([
        rng.uniform(-448, 448, 20000), rng.normal(0, 1, 20000), rng.normal(0, 0.01, 20000),
        rng.uniform(7.4 / 512, 8.1 / 512, 200),
        np.array([oracle.e4m3_decode(i) for i in range(127)]),                      # exact codes
        np.array([(oracle.e4m3_decode(i) + oracle.e4m3_decode(i + 1)) / 2 for i in range(126)]),  # ties
    ]).astype(np.float32)
    xs = np.clip(xs, -448, 448)
    t = torch.from_numpy(xs).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    for x, want in zip(xs.tolist(), t.tolist()):
        got = oracle.e4m3_encode(x)
        if x == 0.0:
            assert got & 0x7F == 0
        elif 7.5 / 512 <= abs(x) < 8.0 / 512:
            assert got & 0x7F == 7 and want & 0x7F == 8, (x, got, want)
        else:
            assert got == want, (x, got, want)


def test_ue8m0_is_pow2(oracle):  # quant.rs:413-423
    assert oracle.ue8m0_decode(127) == 1.0
    assert oracle.ue8m0_decode(128) == 2.0
    assert oracle.ue8m0_decode(126) == 0.5
    assert oracle.ue8m0_decode(0) == 0.0  # the reference's exp2i(-127) clamps the biased exponent to 0
    assert math.isnan(oracle.ue8m0_decode(255))
    assert oracle.ue8m0_encode_pow2(0) == 127
    assert oracle.ue8m0_encode_pow2(3) == 130
    for b in range(1, 255):
        assert oracle.ue8m0_decode(b) == 2.0 ** (b - 127)


def test_bit_tricks_match_reference(oracle):  # quant.rs:425-441
    assert oracle.fast_log2_ceil(1.0) == 0
    assert oracle.fast_log2_ceil(2.0) == 1
    assert oracle.fast_log2_ceil(3.0) == 2
    assert oracle.fast_log2_ceil(0.5) == -1
    assert oracle.fast_log2_ceil(1.5) == 1
    assert oracle.fast_pow2(0) == 1.0
    assert oracle.fast_pow2(3) == 8.0
    assert oracle.fast_pow2(-1) == 0.5
    assert oracle.fast_round_scale(448.0) == 1.0
    assert oracle.fast_round_scale(449.0) == 2.0
    for x in np.random.default_rng(0).uniform(1e-6, 1e4, 500).astype(np.float32).tolist():
        assert oracle.fast_log2_ceil(x) == math.ceil(math.log2(x))


def test_act_quant_fp8_block128_matches_definition(oracle):  # quant.rs:443-466
    x = np.array([(i - 128.0) * 0.7 for i in range(256)], np.float32)
    y, s = oracle.act_quant_fp8(x, 128, False)
    assert s.size == 2
    for b in range(2):
        amax = np.abs(x[b * 128:(b + 1) * 128]).max()
        assert abs(s[b] - amax / 448.0) < 1e-6
    for i in range(256):
        d = oracle.e4m3_decode(int(y[i])) * s[i // 128]
        assert abs(d - x[i]) <= 16.0 * s[i // 128] + 1e-6


def test_act_quant_fp8_block32_pow2_definition(oracle):
    """scale = 2^ceil(log2(amax/448)) and codes = RNE e4m3 of x/scale (closed form via torch)."""
    rng = np.random.default_rng(3)
    x = (rng.normal(0, 1, 64 * 32) * np.repeat(10.0 ** rng.uniform(-3, 3, 64), 32)).astype(np.float32)
    x[32:64] = 0.0  # an all-zero block
    y, s = oracle.act_quant_fp8(x, 32, True)
    for b in range(64):
        blk = x[b * 32:(b + 1) * 32]
        amax = float(np.abs(blk).max())
        if amax == 0:
            assert s[b] == np.float32(2.0 ** -126) and np.all(y[b * 32:(b + 1) * 32] & 0x7F == 0)
            continue
        want_s = 2.0 ** math.ceil(math.log2(np.float32(amax) / np.float32(448.0)))
        assert s[b] == want_s
        q = torch.from_numpy(blk / np.float32(want_s)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        nz = blk != 0
        assert np.array_equal(y[b * 32:(b + 1) * 32][nz], q[nz])
        assert np.abs(blk / want_s).max() <= 448.0


def test_act_quant_fp4_round_scale_is_pow2(oracle):  # quant.rs:468-478
    x = np.array([((i % 7) - 3.0) * 0.9 for i in range(64)], np.float32)
    packed, s = oracle.act_quant_fp4(x, 32, True)
    assert packed.size == 32
    for v in s.tolist():
        e = math.log2(v)
        assert abs(e - round(e)) < 1e-6


def test_dequant_row32_all_codes_all_scales_exact(oracle):
    """Every (code, scale byte) pair against the closed form table[code] * 2^(b-127), in float64."""
    codes = np.arange(16, dtype=np.uint8)
    row = (codes[0::2] | (codes[1::2] << 4)).astype(np.uint8)   # 16 codes -> 8 bytes
    w = np.tile(row, 2)[None, :]                                # one 32-column block
    for b in range(1, 250):
        d = oracle.dequant_fp4_row32(w, np.array([[b]], np.uint8))[0]
        want = np.array(FP4 * 2, np.float64) * 2.0 ** (b - 127)
        assert np.array_equal(d.astype(np.float64), want.astype(np.float32).astype(np.float64))


def test_mxfp4_gemm_exact_in_double(oracle):
    """kernels/cuda/tests_tcgen05_mxf4.cu:25-85 identity: with power-of-two scales every product
    is exact, so a float64 GEMM of the dequantised operands equals the integer-domain sum."""
    rng = np.random.default_rng(5)
    w = rng.integers(0, 256, (8, 32), dtype=np.uint8)
    s = rng.integers(118, 123, (8, 2), dtype=np.uint8)
    d = oracle.dequant_fp4_row32(w, s).astype(np.float64)
    tab = np.array(FP4)
    codes = np.stack([w & 0xF, w >> 4], -1).reshape(8, 64)
    want = tab[codes] * np.repeat(2.0 ** (s.astype(np.float64) - 127), 32, axis=1)
    assert np.array_equal(d, want)
