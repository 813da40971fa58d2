// GPU smoke tests of the C++ HipBackend, written like the reference's own tests: the golden values of
// crates/ferrite-kernel/tests/golden.rs (matmul, swiglu, moe_route) and the fused-MoE parity test of
// crates/ferrite-kernel/tests/gpu_smoke.rs:429-601 (its fixture, its in-test CPU reference, its tolerance),
// plus a capture/replay check (gpu_smoke.rs:268-306).  Usage: hip_backend_smoke <path to libferrite_hip.so>
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <numeric>

#include "hip_backend.hpp"
#include "checkpoint.hpp"

using namespace ferrite;

static int failures = 0;
#define CHECK(cond, ...)                                   \
    do {                                                   \
        if (!(cond)) { ++failures; std::printf("FAIL %s:%d: ", __FILE__, __LINE__); std::printf(__VA_ARGS__); std::printf("\n"); } \
    } while (0)

static Tensor t2(size_t r, size_t c, std::vector<float> v) { return Tensor::from_f32({r, c}, std::move(v)); }

static void matmul_matches_manual(HipBackend& b) {   // golden.rs:14-27
    Tensor x = t2(2, 2, {1, 2, 3, 4}), w = t2(2, 2, {5, 6, 7, 8}), out = Tensor::zeros({2, 2});
    b.matmul(x, w, nullptr, out);
    CHECK(out.data == std::vector<float>({17, 23, 39, 53}), "matmul");
    Tensor bias = t2(1, 2, {0.5f, -0.5f});
    b.matmul(x, w, &bias, out);
    CHECK(out.data == std::vector<float>({17.5f, 22.5f, 39.5f, 52.5f}), "matmul+bias");
    bool threw = false;
    try { Tensor w3 = Tensor::zeros({2, 3}); b.matmul(x, w3, nullptr, out); } catch (const FerriteError& e) { threw = e.kind == FerriteError::ShapeMismatch; }
    CHECK(threw, "k mismatch must be ShapeMismatch");
    threw = false;
    try { Tensor o3 = Tensor::zeros({3, 2}); b.matmul(x, w, nullptr, o3); } catch (const FerriteError& e) { threw = e.kind == FerriteError::InvalidArg; }
    CHECK(threw, "bad out shape must be InvalidArg");
}

static void swiglu_clamps(HipBackend& b) {   // golden.rs:44-55
    Tensor gu = t2(1, 4, {2, 20, 3, 1}), out = Tensor::zeros({1, 2});
    b.swiglu_limited(gu, 10.0f, out);
    float silu2 = 2.0f / (1.0f + std::exp(-2.0f));
    CHECK(std::fabs(out.data[0] - silu2 * 3.0f) < 1e-6f, "swiglu[0]");
    CHECK(std::fabs(out.data[1] - 10.0f / (1.0f + std::exp(-10.0f))) < 1e-6f, "gate clamped to 10");
}

static void rmsnorm_manual(HipBackend& b) {   // golden.rs:30-42
    Tensor x = t2(1, 4, {1, 2, 3, 4}), w = t2(1, 4, {1, 1, 1, 1}), out = Tensor::zeros({1, 4});
    b.rmsnorm(x, w, 1e-6f, out);
    const float mean_sq = (1.0f + 4.0f + 9.0f + 16.0f) / 4.0f, inv = 1.0f / std::sqrt(mean_sq + 1e-6f);
    for (int i = 0; i < 4; ++i) CHECK(std::fabs(out.data[i] - x.data[i] * inv) < 1e-5f, "rmsnorm");
}

static void hc_post_vs_host_loop(HipBackend& b) {   // inputs of gpu_smoke.rs:337-343, loop of cpu.rs:788-807
    const size_t s = 2, n = 4, h = 64;
    Tensor x = Tensor::zeros({s, h}), res = Tensor::zeros({s, n, h}), post = Tensor::zeros({s, n}), comb = Tensor::zeros({s, n, n});
    for (size_t i = 0; i < s * h; ++i) x.data[i] = (float)(i * 7 % 31) * 0.03f;
    for (size_t i = 0; i < s * n * h; ++i) res.data[i] = (float)(i * 13 % 47) * 0.02f - 0.5f;
    for (size_t i = 0; i < s * n; ++i) post.data[i] = 0.25f + 0.2f * (float)i;
    for (size_t i = 0; i < s * n * n; ++i) comb.data[i] = (float)((i * 5 + 3) % 11) / 16.0f;
    Tensor out = b.hc_post(x, res, post, comb);
    bool same = out.shape == std::vector<size_t>{s, n, h};
    for (size_t t = 0; t < s && same; ++t)
        for (size_t i = 0; i < n; ++i)
            for (size_t j = 0; j < h; ++j) {
                volatile float acc = post.data[t * n + i] * x.data[t * h + j];
                for (size_t k = 0; k < n; ++k) {
                    volatile float p = comb.data[(t * n + k) * n + i] * res.data[(t * n + k) * h + j];
                    acc = acc + p;
                }
                if (out.data[(t * n + i) * h + j] != acc) same = false;
            }
    CHECK(same, "hc_post bit-exact against the host loop");
}

static void moe_route_noaux_tc(HipBackend& b) {   // golden.rs:189-210 and gpu_smoke.rs:139-155
    Tensor logits = t2(1, 3, {1.0f, 2.0f, 0.5f}), bias = t2(1, 3, {0, 0, 0.5f});
    Tensor probs = Tensor::zeros({1, 2}), ids = Tensor::zeros({1, 2});
    b.moe_route(logits, bias, 2, 1.0f, probs, ids);
    float s1 = 1.0f / (1.0f + std::exp(-2.0f)), s2 = 1.0f / (1.0f + std::exp(-0.5f));
    CHECK(ids.data[0] == 2.0f && ids.data[1] == 1.0f, "ids %g %g", ids.data[0], ids.data[1]);
    CHECK(std::fabs(probs.data[0] - s2 / (s1 + s2)) < 1e-5f && std::fabs(probs.data[1] - s1 / (s1 + s2)) < 1e-5f, "probs");
    // the tie-free ramp of the reference's GPU test: n=2, e=288, topk=8, scale 2.5
    const size_t n = 2, e = 288, k = 8;
    std::vector<float> lg(n * e), bs(e);
    for (size_t i = 0; i < n * e; ++i) lg[i] = (float)i * 0.017f - 2.0f;
    for (size_t i = 0; i < e; ++i) bs[i] = (float)(i % 11) * 0.01f;
    Tensor L = t2(n, e, lg), B = Tensor::from_f32({e}, bs), P = Tensor::zeros({n, k}), I = Tensor::zeros({n, k});
    b.moe_route(L, B, k, 2.5f, P, I);
    for (size_t r = 0; r < n; ++r) {   // CpuBackend::moe_route restated (cpu.rs:546-569)
        std::vector<float> sig(e);
        std::vector<size_t> order(e);
        for (size_t j = 0; j < e; ++j) { sig[j] = 1.0f / (1.0f + std::exp(-lg[r * e + j])); order[j] = j; }
        std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t c) { return sig[a] + bs[a] > sig[c] + bs[c]; });
        float sum = 0;
        for (size_t q = 0; q < k; ++q) sum += sig[order[q]];
        for (size_t q = 0; q < k; ++q) {
            CHECK(I.data[r * k + q] == (float)order[q], "ramp ids row %zu slot %zu", r, q);
            CHECK(std::fabs(P.data[r * k + q] - sig[order[q]] / (sum + 1.1920929e-7f) * 2.5f) < 1e-5f, "ramp probs");
        }
    }
}

// ---- the fused MoE fixture of gpu_smoke.rs:437-470 ----
static float bex(size_t i, size_t s) { return (float)((i + s) % 4) * 0.25f - 0.5f; }
// encode a matrix with values in {-0.5,-0.25,0,0.25} as MXFP4 with scale 2^-2 (byte 125): value = code * 0.25
static void encode(const std::vector<float>& m, size_t rows, size_t cols, std::vector<uint8_t>& codes, std::vector<uint8_t>& scales) {
    codes.assign(rows * cols / 2, 0);
    scales.assign(rows * cols / 32, 125);
    for (size_t i = 0; i < rows * cols; ++i) {
        float q = m[i] * 4.0f;   // -2, -1, 0, 1
        uint8_t c = q == 0 ? 0 : (q == 1 ? 2 : (q == -1 ? 10 : 12));
        codes[i / 2] |= (i % 2) ? (uint8_t)(c << 4) : c;
    }
}

static void moe_fused_parity(HipBackend& b) {
    const size_t H = 64, I = 32, Is = 16, IsP = 32, E = 8, K = 2;
    const float scaling = 1.2f, limit = 7.0f;
    std::vector<float> x(H), gate_w(E * H), bias(E);
    for (size_t i = 0; i < H; ++i) x[i] = bex(i, 0);
    for (size_t i = 0; i < E * H; ++i) gate_w[i] = bex(i, 5);
    for (size_t i = 0; i < E; ++i) bias[i] = bex(i, 2);
    auto mk = [](size_t r, size_t c, size_t s) { std::vector<float> v(r * c); for (size_t i = 0; i < r * c; ++i) v[i] = bex(i * 7 + s, 0); return v; };
    std::vector<std::vector<float>> eg, eu, ed;
    for (size_t s = 0; s < E; ++s) { eg.push_back(mk(I, H, s * 11)); eu.push_back(mk(I, H, s * 13 + 3)); ed.push_back(mk(H, I, s * 17 + 7)); }
    std::vector<float> sg = mk(Is, H, 29), su = mk(Is, H, 31), sd = mk(H, Is, 37);
    // stack experts; pad the 16-wide shared expert to one 32-wide MXFP4 block with zeros (an exact no-op)
    std::vector<float> G(E * I * H), U(E * I * H), D(E * H * I), SG(IsP * H, 0.f), SU(IsP * H, 0.f), SD(H * IsP, 0.f);
    for (size_t e = 0; e < E; ++e) {
        std::copy(eg[e].begin(), eg[e].end(), G.begin() + e * I * H);
        std::copy(eu[e].begin(), eu[e].end(), U.begin() + e * I * H);
        std::copy(ed[e].begin(), ed[e].end(), D.begin() + e * H * I);
    }
    std::copy(sg.begin(), sg.end(), SG.begin());
    std::copy(su.begin(), su.end(), SU.begin());
    for (size_t h = 0; h < H; ++h) for (size_t i = 0; i < Is; ++i) SD[h * IsP + i] = sd[h * Is + i];
    std::vector<uint8_t> gw, gs, uw, us, dw, ds, sgw, sgs, suw, sus, sdw, sds;
    encode(G, E * I, H, gw, gs); encode(U, E * I, H, uw, us); encode(D, E * H, I, dw, ds);
    encode(SG, IsP, H, sgw, sgs); encode(SU, IsP, H, suw, sus); encode(SD, H, IsP, sdw, sds);
    ferrite_moe_shape shape{(int)H, (int)E, (int)K, (int)I, (int)IsP, 1, 1, scaling, limit};
    MoeHostWeights hw{gate_w.data(), bias.data(), gw.data(), gs.data(), uw.data(), us.data(), dw.data(), ds.data(),
                      sgw.data(), sgs.data(), suw.data(), sus.data(), sdw.data(), sds.data()};
    MoeLayerDev layer = b.load_moe_layer(shape, hw);
    DevBuf dx(H * 4), dout(H * 4);
    dx.upload(x.data(), H * 4);
    b.moe_layer_dev_mxfp4(layer, dx, FERRITE_DT_F32, 1, dout, FERRITE_DT_F32, FERRITE_MODE_F32_CHECK);
    b.sync();
    std::vector<float> hv(H);
    dout.download(hv.data(), H * 4);

    // CPU reference spelled out as in gpu_smoke.rs:493-562
    std::vector<float> logits(E), scores(E), choice(E);
    for (size_t j = 0; j < E; ++j) { float s = 0; for (size_t k = 0; k < H; ++k) s += x[k] * gate_w[j * H + k]; logits[j] = s; }
    for (size_t j = 0; j < E; ++j) { scores[j] = 1.0f / (1.0f + std::exp(-logits[j])); choice[j] = scores[j] + bias[j]; }
    std::vector<size_t> order(E);
    std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t c) { return choice[a] > choice[c]; });
    float rsum = scores[order[0]] + scores[order[1]];
    auto silu = [](float g) { return g / (1.0f + std::exp(-g)); };
    std::vector<float> ref(H, 0.f);
    auto run_expert = [&](const std::vector<float>& g, const std::vector<float>& u, const std::vector<float>& d, size_t inter, float wgt) {
        std::vector<float> act(inter);
        for (size_t i = 0; i < inter; ++i) {
            float gv = 0, uv = 0;
            for (size_t k = 0; k < H; ++k) { gv += x[k] * g[i * H + k]; uv += x[k] * u[i * H + k]; }
            gv = std::fmin(gv, limit);
            uv = std::fmin(std::fmax(uv, -limit), limit);
            act[i] = silu(gv) * uv;
        }
        for (size_t h = 0; h < H; ++h) { float y = 0; for (size_t i = 0; i < inter; ++i) y += act[i] * d[h * inter + i]; ref[h] += wgt * y; }
    };
    for (size_t jj = 0; jj < K; ++jj) run_expert(eg[order[jj]], eu[order[jj]], ed[order[jj]], I, scores[order[jj]] / rsum * scaling);
    run_expert(sg, su, sd, Is, 1.0f);
    float maxd = 0;
    for (size_t i = 0; i < H; ++i) maxd = std::fmax(maxd, std::fabs(hv[i] - ref[i]));
    CHECK(maxd < 1e-4f, "moe_fused mismatch: max diff %g (tol 1e-4)", maxd);
    std::printf("[moe-fused] parity max_diff %g (ids %zu %zu)\n", maxd, order[0], order[1]);
}

static void graph_capture_smoke(HipBackend& b) {   // gpu_smoke.rs:268-306: capture, replay, same result as eager
    const int H = 256, I = 128, E = 8, K = 2, n = 24;
    ferrite_moe_shape shape{H, E, K, I, I, 4, 2, 2.5f, 10.0f};
    uint64_t st = 0x9E3779B97F4A7C15ull;
    auto rnd = [&]() { st ^= st >> 12; st ^= st << 25; st ^= st >> 27; return st * 0x2545F4914F6CDD1Dull; };   // xorshift64*
    auto bytes = [&](size_t nb) { std::vector<uint8_t> v(nb); for (auto& c : v) c = (uint8_t)(rnd() >> 56); return v; };
    auto scl = [&](size_t nb) { std::vector<uint8_t> v(nb); for (auto& c : v) c = 119 + (uint8_t)((rnd() >> 60) & 1); return v; };
    std::vector<float> rw((size_t)E * H), rb(E);
    for (auto& v : rw) v = ((float)(rnd() >> 40) / 16777216.0f - 0.5f) * 0.1f;
    for (auto& v : rb) v = ((float)(rnd() >> 40) / 16777216.0f - 0.5f) * 0.02f;
    auto gw = bytes((size_t)E * I * H / 2), uw = bytes((size_t)E * I * H / 2), dw = bytes((size_t)E * H * I / 2);
    auto gs = scl((size_t)E * I * H / 32), us = scl((size_t)E * I * H / 32), ds = scl((size_t)E * H * I / 32);
    auto sgw = bytes((size_t)I * H / 2), suw = bytes((size_t)I * H / 2), sdw = bytes((size_t)H * I / 2);
    auto sgs = scl((size_t)I * H / 32), sus = scl((size_t)I * H / 32), sds = scl((size_t)H * I / 32);
    MoeHostWeights hw{rw.data(), rb.data(), gw.data(), gs.data(), uw.data(), us.data(), dw.data(), ds.data(),
                      sgw.data(), sgs.data(), suw.data(), sus.data(), sdw.data(), sds.data()};
    MoeLayerDev layer = b.load_moe_layer(shape, hw);
    DevBuf dx((size_t)n * H * 4), dout((size_t)n * H * 4), deager((size_t)n * H * 4);
    std::vector<float> x((size_t)n * H);
    auto fill = [&]() { for (auto& v : x) v = ((float)(rnd() >> 40) / 16777216.0f - 0.5f) * 4.0f; };
    fill();
    dx.upload(x.data(), x.size() * 4);
    b.moe_layer_dev_mxfp4(layer, dx, FERRITE_DT_F32, n, dout, FERRITE_DT_F32, FERRITE_MODE_MFMA_FP8);   // warm
    b.sync();
    b.begin_capture();
    b.moe_layer_dev_mxfp4(layer, dx, FERRITE_DT_F32, n, dout, FERRITE_DT_F32, FERRITE_MODE_MFMA_FP8);
    OpTrace trace = b.end_capture();
    CHECK(trace.len() == 1 && trace.ops[0].op == "moe_layer_mxfp4", "trace ops");
    std::vector<float> a((size_t)n * H), c((size_t)n * H);
    for (int rep = 0; rep < 3; ++rep) {
        fill();
        dx.upload(x.data(), x.size() * 4);
        b.moe_layer_dev_mxfp4(layer, dx, FERRITE_DT_F32, n, deager, FERRITE_DT_F32, FERRITE_MODE_MFMA_FP8);
        b.sync();
        b.begin_verify(trace);
        CHECK(b.end_verify(), "replay failed");
        dout.download(a.data(), a.size() * 4);
        deager.download(c.data(), c.size() * 4);
        CHECK(std::memcmp(a.data(), c.data(), a.size() * 4) == 0, "replay %d differs from eager", rep);
    }
    b.graph_destroy(trace);
}

// A shard written here (safetensors: 8-byte header length, JSON header, tensors back to back) is streamed by the
// checkpoint loader into a packed buffer that must equal, byte for byte, the one load_moe_layer builds from the
// same tensors in memory (the names are those of crates/ferrite-models/src/dsv41/weights.rs:333-341).
static void checkpoint_loader_roundtrip(HipBackend& b, const std::string& so_path) {
    const size_t H = 256, I = 128, Is = 128, E = 3;
    ferrite_moe_shape shape{(int)H, (int)E, 2, (int)I, (int)Is, 1, 1, 1.0f, 7.0f};
    uint32_t rng = 12345u;
    auto fill = [&](std::vector<uint8_t>& v, size_t n, bool scale) {
        v.resize(n);
        for (auto& x : v) { rng = rng * 1664525u + 1013904223u; x = scale ? (uint8_t)(118 + (rng >> 28)) : (uint8_t)(rng >> 24); }
    };
    std::vector<float> router(E * H), bias(E);
    for (size_t i = 0; i < E * H; ++i) router[i] = bex(i, 3);
    for (size_t i = 0; i < E; ++i) bias[i] = bex(i, 1);
    std::vector<uint8_t> gw, gs, uw, us, dw, ds, sgw, sgs, suw, sus, sdw, sds;
    fill(gw, E * I * H / 2, false); fill(gs, E * I * H / 32, true); fill(uw, E * I * H / 2, false); fill(us, E * I * H / 32, true);
    fill(dw, E * H * I / 2, false); fill(ds, E * H * I / 32, true);
    fill(sgw, Is * H / 2, false); fill(sgs, Is * H / 32, true); fill(suw, Is * H / 2, false); fill(sus, Is * H / 32, true);
    fill(sdw, H * Is / 2, false); fill(sds, H * Is / 32, true);
    MoeHostWeights hw{router.data(), bias.data(), gw.data(), gs.data(), uw.data(), us.data(), dw.data(), ds.data(),
                      sgw.data(), sgs.data(), suw.data(), sus.data(), sdw.data(), sds.data()};
    MoeLayerDev mem = b.load_moe_layer(shape, hw);

    std::string header = "{";
    std::string blob;
    auto add = [&](const std::string& name, const char* dtype, size_t r, size_t c, const void* data, size_t bytes) {
        if (header.size() > 1) header += ",";
        header += "\"" + name + "\":{\"dtype\":\"" + dtype + "\",\"shape\":[" + std::to_string(r) +
                  (c ? "," + std::to_string(c) : std::string()) + "],\"data_offsets\":[" + std::to_string(blob.size()) + "," +
                  std::to_string(blob.size() + bytes) + "]}";
        blob.append(static_cast<const char*>(data), bytes);
    };
    const std::string p = "layers.6.ffn";
    add(p + ".gate.weight", "F32", E, H, router.data(), E * H * 4);
    add(p + ".gate.bias", "F32", E, 0, bias.data(), E * 4);
    for (size_t e = 0; e <= E; ++e) {
        const bool sh = e == E;
        const std::string q = sh ? p + ".shared_experts" : p + ".experts." + std::to_string(e);
        const size_t inter = sh ? Is : I;
        const size_t cw = inter * H / 2, cs = inter * H / 32;
        add(q + ".w1.weight", "I8", inter, H / 2, (sh ? sgw.data() : gw.data() + e * cw), cw);
        add(q + ".w1.scale", "F8_E8M0", inter, H / 32, (sh ? sgs.data() : gs.data() + e * cs), cs);
        add(q + ".w2.weight", "I8", H, inter / 2, (sh ? sdw.data() : dw.data() + e * cw), cw);
        add(q + ".w2.scale", "F8_E8M0", H, inter / 32, (sh ? sds.data() : ds.data() + e * cs), cs);
        add(q + ".w3.weight", "I8", inter, H / 2, (sh ? suw.data() : uw.data() + e * cw), cw);
        add(q + ".w3.scale", "F8_E8M0", inter, H / 32, (sh ? sus.data() : us.data() + e * cs), cs);
    }
    header += "}";
    while (header.size() % 8) header += ' ';
    char path[] = "/tmp/ferrite_smoke_XXXXXX";
    const int fd = mkstemp(path);
    CHECK(fd >= 0, "mkstemp failed");
    if (fd < 0) return;
    FILE* f = fdopen(fd, "wb");
    const uint64_t hlen = header.size();
    fwrite(&hlen, 8, 1, f);
    fwrite(header.data(), 1, header.size(), f);
    fwrite(blob.data(), 1, blob.size(), f);
    fclose(f);

    SafetensorsIndex index = SafetensorsIndex::read_header(path);
    const auto missing = index.validate(moe_layer_specs(MoeNaming::Dsv41, p, shape));
    CHECK(missing.empty(), "validate reports %zu missing tensors (first: %s)", missing.size(), missing.empty() ? "" : missing[0].c_str());
    CHECK(index.tensors.size() == 2 + 6 * (E + 1), "index holds %zu tensors", index.tensors.size());
    MappedFile file(path);
    MoeCheckpointLoader loader(so_path, 0);
    const size_t pb = loader.packed_bytes(shape);
    CHECK(pb == mem.packed.bytes, "packed size %zu vs %zu", pb, mem.packed.bytes);
    DevBuf packed(pb), dbias(E * 4);
    LoadOptions opt;
    opt.workers = 3;
    opt.pad_scale_rows = true;
    const LoadStats st = loader.load_layer(file, index, MoeNaming::Dsv41, p, shape, static_cast<uint8_t*>(packed.ptr),
                                           static_cast<float*>(dbias.ptr), opt);
    std::vector<uint8_t> a(pb), c(pb);
    packed.download(a.data(), pb);
    mem.packed.download(c.data(), pb);
    CHECK(std::memcmp(a.data(), c.data(), pb) == 0, "packed buffer from the shard differs from the memory-loaded one");
    std::vector<float> hb(E);
    dbias.download(hb.data(), E * 4);
    CHECK(std::memcmp(hb.data(), bias.data(), E * 4) == 0, "routing bias differs");
    bool threw = false;
    try {
        loader.load_layer(file, index, MoeNaming::Dsv41, "layers.7.ffn", shape, static_cast<uint8_t*>(packed.ptr),
                          static_cast<float*>(dbias.ptr), opt);
    } catch (const FerriteError& e) {
        threw = std::string(e.what()).find("missing tensor layers.7.ffn.gate.weight") != std::string::npos;
    }
    CHECK(threw, "a missing layer must be reported by name");
    std::remove(path);
    std::printf("[checkpoint] %llu source bytes -> %llu packed, %d workers\n", (unsigned long long)st.source_bytes,
                (unsigned long long)st.packed_bytes, st.workers);
}

int main(int argc, char** argv) {
    if (argc < 2) { std::printf("usage: %s libferrite_hip.so\n", argv[0]); return 2; }
    try {
        HipBackend b(argv[1], 0);
        std::printf("build id %s\n", b.build_id().c_str());
        matmul_matches_manual(b); std::printf("matmul ok\n"); std::fflush(stdout);
        swiglu_clamps(b); std::printf("swiglu ok\n"); std::fflush(stdout);
        rmsnorm_manual(b); std::printf("rmsnorm ok\n"); std::fflush(stdout);
        hc_post_vs_host_loop(b); std::printf("hc_post ok\n"); std::fflush(stdout);
        moe_route_noaux_tc(b); std::printf("moe_route ok\n"); std::fflush(stdout);
        moe_fused_parity(b); std::fflush(stdout);
        graph_capture_smoke(b); std::printf("graph ok\n"); std::fflush(stdout);
        checkpoint_loader_roundtrip(b, argv[1]); std::printf("checkpoint ok\n");
    } catch (const std::exception& e) {
        std::printf("EXCEPTION: %s\n", e.what());
        return 1;
    }
    std::printf(failures ? "FAILED (%d)\n" : "ALL OK\n", failures);
    return failures ? 1 : 0;
}
