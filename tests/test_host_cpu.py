"""CPU-side checks of the product: the C ABI library loads and exports every symbol the header declares, the
op recorder behaves like the reference's (crates/ferrite-kernel/src/graph.rs:85-165), and the scalar numerics the
kernels are built from (csrc/numerics.hpp, compiled for the host) agree with libm / the oracle bit for bit."""
import ctypes as C
import math
import os
import re
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from ferrite_amd import backend
    hdr = open(os.path.join(ROOT, "include", "ferrite_hip.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = sorted(set(re.findall(r"\b(ferrite_[a-z0-9_]+)\s*\(", hdr)))
    assert len(declared) >= 20
    lib = backend.load_library()
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in ferrite_hip.h but not exported"
    assert sorted(backend.EXPORTS) == declared
    assert lib.ferrite_kernel_abi_version() == backend.ABI_VERSION
    assert lib.ferrite_kernel_build_id().decode().startswith("ferrite-hip-")


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more it says so and exits before touching a device."""
    for extra_env in ({}, {"WORLD_SIZE": "2"}):
        env = dict(os.environ, **extra_env)
        args = [os.sys.executable, os.path.join(ROOT, "bench.py")] + ([] if extra_env else ["--gpus", "2"])
        res = subprocess.run(args, capture_output=True, text=True, env=env, timeout=60)
        assert res.returncode == 2
        assert "one GPU" in res.stderr and res.stdout == ""


def _layer_rc(lib, backend, n, **over):
    """Return code of the layer call for a shape; argument checks run before any pointer is used or any GPU call is
    made, so dummy non-null pointers do on a machine without a GPU."""
    base = dict(hidden=256, n_experts=64, topk=4, inter=128, shared_inter=128, n_group=4, topk_group=2,
                routed_scaling=2.5, swiglu_limit=10.0)
    base.update(over)
    shape = backend.MoeShape(*[base[k] for k, _ in backend.MoeShape._fields_])
    w = backend.MoeWeights()
    dummy = C.c_void_p(4096)
    return lib.ferrite_moe_layer_mxfp4(C.byref(shape), C.byref(w), dummy, dummy, backend.DT_F32, n, dummy,
                                       backend.DT_F32, backend.MODE_MFMA_FP8, dummy, 1 << 30, None)


def test_layer_refuses_routing_parameters_outside_the_kernels_limits():
    """The fused head (decode-sized batches) and the separate routing launches refuse the same parameters, up front:
    what ferrite_moe_route returns for them, at 32 tokens as at 4096."""
    from ferrite_amd import backend
    lib = backend.load_library()
    for n in (32, 4096):
        assert _layer_rc(lib, backend, n, n_experts=64, topk=33, n_group=1, topk_group=1) == backend.DECLINED
        assert _layer_rc(lib, backend, n, n_experts=130, topk=4, n_group=65, topk_group=33) == backend.DECLINED
        assert _layer_rc(lib, backend, n, n_experts=66, topk=4, n_group=4, topk_group=2) == backend.ERR_INVALID_ARG
        assert _layer_rc(lib, backend, n, n_experts=64, topk=4, n_group=4, topk_group=0) == backend.ERR_INVALID_ARG
        assert _layer_rc(lib, backend, n, n_experts=64, topk=40, n_group=4, topk_group=2) == backend.ERR_INVALID_ARG
        assert _layer_rc(lib, backend, n, n_experts=1024, topk=4, n_group=1, topk_group=1) == backend.DECLINED
    # more tokens than a launch's grid.y takes: refused before anything is enqueued, not half way through
    assert _layer_rc(lib, backend, 65536) == backend.DECLINED
    assert _layer_rc(lib, backend, 0) == backend.ERR_INVALID_ARG


def test_static_workspace_entry_refuses_oversize_before_touching_a_gpu():
    """The size check of ferrite_moe_layer_mxfp4_static is host arithmetic: it answers without a GPU."""
    from ferrite_amd import backend
    lib = backend.load_library()
    shape = backend.MoeShape(4096, 128, 8, 1536, 1536, 8, 4, 2.5, 10.0)
    w = backend.MoeWeights()
    d = C.c_void_p(4096)
    need = lib.ferrite_moe_layer_workspace_bytes(C.byref(shape), 192, backend.MODE_MFMA_FP8)
    assert need > backend.STATIC_WORKSPACE_BYTES
    rc = lib.ferrite_moe_layer_mxfp4_static(C.byref(shape), C.byref(w), d, d, backend.DT_BF16, 192, d, backend.DT_BF16,
                                            backend.MODE_MFMA_FP8, None)
    assert rc == backend.ERR_WORKSPACE
    msg = lib.ferrite_hip_last_error().decode()
    assert str(need) in msg and str(backend.STATIC_WORKSPACE_BYTES) in msg
    assert lib.ferrite_moe_layer_workspace_bytes(C.byref(shape), 32, backend.MODE_MFMA_FP8) <= backend.STATIC_WORKSPACE_BYTES
    hdr = open(os.path.join(ROOT, "include", "ferrite_hip.h")).read()
    assert "#define FERRITE_STATIC_WORKSPACE_BYTES (16u << 20)" in hdr and backend.STATIC_WORKSPACE_BYTES == 16 << 20


def test_overrides_validate_their_arguments():
    from ferrite_amd import backend
    lib = backend.load_library()
    assert lib.ferrite_hip_set_override(backend.OVERRIDE_UNIT_ROWS, 64) == backend.ERR_INVALID_ARG
    assert lib.ferrite_hip_set_override(backend.OVERRIDE_Y_F32, 2) == backend.ERR_INVALID_ARG
    assert lib.ferrite_hip_set_override(7, 0) == backend.ERR_INVALID_ARG
    shape = backend.MoeShape(4096, 128, 8, 1536, 1536, 8, 4, 2.5, 10.0)
    assert lib.ferrite_moe_layer_unit_rows(C.byref(shape), 32, backend.MODE_MFMA_FP8) == 16
    assert lib.ferrite_moe_layer_unit_rows(C.byref(shape), 4096, backend.MODE_MFMA_FP8) == 128
    assert lib.ferrite_hip_set_override(backend.OVERRIDE_UNIT_ROWS, 128) == backend.OK
    assert lib.ferrite_moe_layer_unit_rows(C.byref(shape), 32, backend.MODE_MFMA_FP8) == 128
    assert lib.ferrite_hip_set_override(backend.OVERRIDE_UNIT_ROWS, 0) == backend.OK
    assert lib.ferrite_moe_layer_unit_rows(C.byref(shape), 32, backend.MODE_MFMA_FP8) == 16


def test_layer_check_answers_without_a_gpu_and_units_follow_mode_and_size():
    """ferrite_moe_layer_check is host arithmetic: what a layer call would answer before it enqueues anything.  The
    MFMA modes decline sizes that are not multiples of 128 (the f32 mode takes them: the order the host mirrors fall
    back in); two-term activations are served at every batch size, on 16-row units for decode-sized batches and on
    64-row units (128 with one term) for prefill-sized ones; a declined call has no workspace size."""
    from ferrite_amd import backend
    lib = backend.load_library()
    shape = backend.MoeShape(4096, 128, 8, 1536, 1536, 8, 4, 2.5, 10.0)
    for n in (32, 192, 4096):
        for mode in (backend.MODE_F32_CHECK, backend.MODE_MFMA_FP8, backend.MODE_MFMA_FP8_X2):
            assert lib.ferrite_moe_layer_check(C.byref(shape), n, mode) == backend.OK
    rows = lambda n, mode: lib.ferrite_moe_layer_unit_rows(C.byref(shape), n, mode)
    assert [rows(n, backend.MODE_MFMA_FP8) for n in (32, 192, 255, 256, 4096)] == [16, 16, 16, 128, 128]
    assert [rows(n, backend.MODE_MFMA_FP8_X2) for n in (32, 192, 255, 256, 4096)] == [16, 16, 16, 64, 64]
    assert lib.ferrite_hip_set_override(backend.OVERRIDE_UNIT_ROWS, 128) == backend.OK
    assert rows(32, backend.MODE_MFMA_FP8_X2) == 64 and rows(32, backend.MODE_MFMA_FP8) == 128
    assert lib.ferrite_hip_set_override(backend.OVERRIDE_UNIT_ROWS, 16) == backend.OK
    assert rows(4096, backend.MODE_MFMA_FP8_X2) == 16
    assert lib.ferrite_hip_set_override(backend.OVERRIDE_UNIT_ROWS, 0) == backend.OK
    sz = lambda n, mode: lib.ferrite_moe_layer_workspace_bytes(C.byref(shape), n, mode)
    assert sz(4096, backend.MODE_MFMA_FP8_X2) > sz(4096, backend.MODE_MFMA_FP8) > 0      # the second planes
    odd = backend.MoeShape(160, 8, 3, 96, 64, 4, 2, 2.5, 10.0)
    for n in (20, 200):
        assert lib.ferrite_moe_layer_check(C.byref(odd), n, backend.MODE_MFMA_FP8_X2) == backend.DECLINED
        assert lib.ferrite_moe_layer_check(C.byref(odd), n, backend.MODE_MFMA_FP8) == backend.DECLINED
        assert lib.ferrite_moe_layer_check(C.byref(odd), n, backend.MODE_F32_CHECK) == backend.OK
        assert sz(n, backend.MODE_MFMA_FP8) > 0
        assert lib.ferrite_moe_layer_workspace_bytes(C.byref(odd), n, backend.MODE_MFMA_FP8) == 0
    assert lib.ferrite_moe_layer_check(C.byref(shape), 32, 9) == backend.ERR_INVALID_ARG
    assert lib.ferrite_moe_layer_check(None, 32, backend.MODE_MFMA_FP8) == backend.ERR_INVALID_ARG


def test_library_sources_read_no_environment():
    """Launchers may be recorded into a stream capture; the reference reads its gates once for that reason
    (cuda.rs:5730-5731).  Here no source of the library reads the environment at all."""
    csrc = os.path.join(ROOT, "ferrite_amd", "csrc")
    for name in sorted(os.listdir(csrc)):
        text = open(os.path.join(csrc, name)).read()
        assert "getenv" not in text, name


def test_backend_refuses_to_run_without_gpu_or_library(tmp_path):
    import torch
    from ferrite_amd import backend
    with pytest.raises(backend.FerriteError):
        backend.load_library(str(tmp_path / "missing.so"))
    if not torch.cuda.is_available():
        with pytest.raises(backend.FerriteError):
            backend.HipBackend()


def test_recorder_capture_and_verify():  # graph.rs:141-165
    from ferrite_amd.backend import Recorder
    r = Recorder()
    r.begin_capture()
    r.record("matmul", [[4, 8], [16, 8]])
    r.record("rmsnorm", [[4, 8]])
    trace = r.end_capture()
    assert len(trace) == 2
    r.begin_verify(trace)
    r.record("matmul", [[4, 8], [16, 8]])
    r.record("rmsnorm", [[4, 8]])
    assert r.end_verify()
    r.begin_verify(trace)
    r.record("matmul", [[4, 8], [16, 8]])
    r.record("rmsnorm", [[4, 8]])
    r.record("matmul", [[4, 8], [16, 8]])
    assert not r.end_verify()
    r.begin_verify(trace)
    r.record("matmul", [[8, 8], [16, 8]])
    r.record("rmsnorm", [[8, 8]])
    assert not r.end_verify()
    assert not r.end_verify()          # not verifying: false, like the reference
    r.record("matmul")                 # Off: ignored
    assert r.ops == []


@pytest.fixture(scope="module")
def shim(tmp_path_factory):
    out = tmp_path_factory.mktemp("shim") / "libnumerics_shim.so"
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off", "-o", str(out),
                           os.path.join(ROOT, "tests", "numerics_host_shim.cpp")])
    lib = C.CDLL(str(out))
    for f in ("shim_expf", "shim_sigmoid", "shim_e4m3_decode", "shim_e2m1_decode", "shim_ue8m0_decode"):
        getattr(lib, f).restype = C.c_float
    lib.shim_expf.argtypes = [C.c_float]
    lib.shim_sigmoid.argtypes = [C.c_float]
    lib.shim_swiglu.restype = C.c_float
    lib.shim_swiglu.argtypes = [C.c_float] * 3
    lib.shim_e4m3_encode.argtypes = [C.c_float]
    lib.shim_block_scale_e8m0.argtypes = [C.c_float]
    lib.shim_e4m3_decode.argtypes = [C.c_uint]
    lib.shim_e2m1_decode.argtypes = [C.c_uint]
    lib.shim_ue8m0_decode.argtypes = [C.c_uint]
    lib.shim_expf_many.argtypes = [C.c_void_p, C.c_void_p, C.c_long]
    return lib


def libm_expf(x: np.ndarray) -> np.ndarray:
    libm = C.CDLL("libm.so.6")
    libm.expf.restype = C.c_float
    libm.expf.argtypes = [C.c_float]
    return np.array([libm.expf(float(v)) for v in x], np.float32)


def test_expf_port_is_bit_identical_to_libm(shim):
    """fe_expf restates glibc's expf; every sampled float must round to the same bits."""
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.uniform(-104, 89, 200000), rng.normal(0, 3, 200000), rng.uniform(-1e-3, 1e-3, 20000),
        np.array([0.0, -0.0, 1.0, -1.0, 88.0, 88.5, 88.72, 88.73, 89.0, -87.3, -88.0, -103.0, -103.9, -104.0, -150.0,
                  1e-30, -1e-30, np.inf, -np.inf, 0.5, -0.5, 10.0, -10.0, 17.3])]).astype(np.float32)
    # plus a stride through the raw bit patterns of the interesting range
    bits = np.arange(0x3C000000, 0x42B00000, 3571, dtype=np.uint32)
    xs = np.concatenate([xs, bits.view(np.float32), -bits.view(np.float32)])
    got = np.empty_like(xs)
    shim.shim_expf_many(xs.ctypes.data, got.ctypes.data, xs.size)
    want = libm_expf(xs)
    neq = np.nonzero(got.view(np.uint32) != want.view(np.uint32))[0]
    assert neq.size == 0, [(float(xs[i]), float(got[i]), float(want[i])) for i in neq[:5]]
    assert math.isnan(shim.shim_expf(float("nan")))


def test_sigmoid_and_swiglu_match_the_oracle(shim, oracle):
    rng = np.random.default_rng(1)
    g = rng.normal(0, 5, 4000).astype(np.float32)
    u = rng.normal(0, 5, 4000).astype(np.float32)
    g[:4] = [20.0, -200.0, 95.0, 10.0]
    want = oracle.swiglu_limited(np.concatenate([g, u])[None, :], 10.0)[0]
    got = np.array([shim.shim_swiglu(float(a), float(b), 10.0) for a, b in zip(g, u)], np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    logits = rng.normal(0, 3, (1, 512)).astype(np.float32)
    probs, ids = oracle.moe_route(logits, np.zeros(512, np.float32), 1, 1.0)
    # with topk = 1 the reference's weight is sig/(sig+eps): recompute it from the shim's sigmoid
    j = int(ids[0, 0])
    s = np.float32(shim.shim_sigmoid(float(logits[0, j])))
    assert probs[0, 0] == np.float32(np.float32(s / np.float32(s + np.finfo(np.float32).eps)) * np.float32(1.0))


def test_format_primitives_match_the_oracle(shim, oracle):
    for b in range(256):
        if b & 0x7F != 0x7F:
            assert shim.shim_e4m3_decode(b) == oracle.e4m3_decode(b)
        d = shim.shim_ue8m0_decode(b)
        assert (math.isnan(d) and b == 255) or d == oracle.ue8m0_decode(b)
    for c in range(16):
        assert shim.shim_e2m1_decode(c) == oracle.e2m1_decode(c)
    rng = np.random.default_rng(2)
    xs = np.concatenate([rng.uniform(-500, 500, 20000), rng.normal(0, 1, 20000), rng.uniform(-0.02, 0.02, 20000),
                         np.array([0.0, -0.0, 448.0, 449.0, 7.5 / 512, 7.49 / 512, 8.0 / 512, 2.0 ** -6, 1e9, -1e9,
                                   np.inf, -np.inf])]).astype(np.float32)
    for x in xs.tolist():
        assert shim.shim_e4m3_encode(x) == oracle.e4m3_encode(x), x
    for a in np.concatenate([10.0 ** rng.uniform(-30, 30, 2000), [0.0, 448.0, 449.0, 224.0, 1e-45]]).astype(np.float32).tolist():
        byte = shim.shim_block_scale_e8m0(a)
        _, s = oracle.act_quant_fp8(np.array([a] + [0.0] * 31, np.float32), 32, True)
        assert 2.0 ** (byte - 127) == float(s[0]), a
