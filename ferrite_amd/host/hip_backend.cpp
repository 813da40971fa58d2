#include "hip_backend.hpp"

#include <dlfcn.h>
#include <hip/hip_runtime_api.h>

#include <cstring>

namespace ferrite {

static void hipck(hipError_t e, const char* what) {
    if (e != hipSuccess)
        throw FerriteError(FerriteError::InvalidArg, std::string("HIP ") + what + ": " + hipGetErrorString(e));
}

Tensor Tensor::zeros(std::vector<size_t> shape, DType dt) {
    Tensor t;
    t.shape = std::move(shape);
    t.dtype = dt;
    t.data.assign(t.numel(), 0.0f);
    return t;
}
Tensor Tensor::from_f32(std::vector<size_t> shape, std::vector<float> v) {
    Tensor t;
    t.shape = std::move(shape);
    t.data = std::move(v);
    if (t.data.size() != t.numel()) throw FerriteError(FerriteError::ShapeMismatch, "from_f32: data/shape mismatch");
    return t;
}
size_t Tensor::numel() const {
    size_t n = 1;
    for (size_t d : shape) n *= d;
    return n;
}

DevBuf::DevBuf(size_t nbytes) : bytes(nbytes) { hipck(hipMalloc(&ptr, nbytes ? nbytes : 16), "hipMalloc"); }
DevBuf::~DevBuf() {
    if (ptr) (void)hipFree(ptr);
}
DevBuf& DevBuf::operator=(DevBuf&& o) noexcept {
    if (this != &o) {
        if (ptr) (void)hipFree(ptr);
        ptr = o.ptr; bytes = o.bytes;
        o.ptr = nullptr; o.bytes = 0;
    }
    return *this;
}
void DevBuf::upload(const void* src, size_t nbytes) {
    if (nbytes > bytes) throw FerriteError(FerriteError::IndexOutOfBounds, "upload larger than buffer");
    hipck(hipMemcpy(ptr, src, nbytes, hipMemcpyHostToDevice), "hipMemcpy H2D");
}
void DevBuf::download(void* dst, size_t nbytes) const {
    if (nbytes > bytes) throw FerriteError(FerriteError::IndexOutOfBounds, "download larger than buffer");
    hipck(hipMemcpy(dst, ptr, nbytes, hipMemcpyDeviceToHost), "hipMemcpy D2H");
}

struct HipBackend::Api {
#define FN(name) decltype(&::name) name = nullptr
    FN(ferrite_kernel_build_id); FN(ferrite_kernel_abi_version); FN(ferrite_hip_last_error); FN(ferrite_hip_warmup);
    FN(ferrite_matmul_f32); FN(ferrite_swiglu_limited_f32); FN(ferrite_moe_route);
    FN(ferrite_rmsnorm_f32); FN(ferrite_hc_post_f32);
    FN(ferrite_moe_packed_bytes); FN(ferrite_moe_pack_weights);
    FN(ferrite_moe_layer_workspace_bytes); FN(ferrite_moe_layer_workspace_init); FN(ferrite_moe_layer_mxfp4);
    FN(ferrite_moe_layer_check);
    FN(ferrite_graph_begin); FN(ferrite_graph_end); FN(ferrite_graph_launch); FN(ferrite_graph_destroy);
#undef FN
};

HipBackend::HipBackend(const std::string& so_path, int device) : api_(new Api) {
    so_ = dlopen(so_path.c_str(), RTLD_NOW | RTLD_LOCAL);
    if (!so_) throw FerriteError(FerriteError::InvalidArg, std::string("dlopen ") + so_path + ": " + dlerror());
#define LOAD(name)                                                                              \
    api_->name = reinterpret_cast<decltype(api_->name)>(dlsym(so_, #name));                      \
    if (!api_->name) throw FerriteError(FerriteError::InvalidArg, "missing symbol " #name)
    LOAD(ferrite_kernel_build_id); LOAD(ferrite_kernel_abi_version); LOAD(ferrite_hip_last_error);
    LOAD(ferrite_hip_warmup);
    LOAD(ferrite_matmul_f32); LOAD(ferrite_swiglu_limited_f32); LOAD(ferrite_moe_route);
    LOAD(ferrite_rmsnorm_f32); LOAD(ferrite_hc_post_f32);
    LOAD(ferrite_moe_packed_bytes); LOAD(ferrite_moe_pack_weights);
    LOAD(ferrite_moe_layer_workspace_bytes); LOAD(ferrite_moe_layer_workspace_init); LOAD(ferrite_moe_layer_mxfp4);
    LOAD(ferrite_moe_layer_check);
    LOAD(ferrite_graph_begin); LOAD(ferrite_graph_end); LOAD(ferrite_graph_launch); LOAD(ferrite_graph_destroy);
#undef LOAD
    if (api_->ferrite_kernel_abi_version() != FERRITE_ABI_VERSION)
        throw FerriteError(FerriteError::InvalidArg, "libferrite_hip.so ABI version mismatch");
    hipck(hipSetDevice(device), "hipSetDevice");
    hipStream_t s;
    hipck(hipStreamCreate(&s), "hipStreamCreate");   // one stream per backend, default priority
    stream_ = s;
    ck(api_->ferrite_hip_warmup(), "warmup");   // LDS limits, before anything is captured
}

HipBackend::~HipBackend() {
    if (stream_) (void)hipStreamDestroy(static_cast<hipStream_t>(stream_));
    if (so_) dlclose(so_);
}

std::string HipBackend::build_id() const { return api_->ferrite_kernel_build_id(); }

void HipBackend::ck(int rc, const char* what) const {
    if (rc == FERRITE_OK) return;
    if (rc == FERRITE_DECLINED) throw FerriteError(FerriteError::InvalidArg, std::string("HIP ") + what + ": shape declined");
    throw FerriteError(FerriteError::InvalidArg,
                       std::string("HIP ") + what + ": rc=" + std::to_string(rc) + " " + api_->ferrite_hip_last_error());
}

void HipBackend::rec(const char* op) {
    if (capturing_) recorded_.push_back(OpRecord{op, {}});
}

void HipBackend::sync() { hipck(hipStreamSynchronize(static_cast<hipStream_t>(stream_)), "hipStreamSynchronize"); }

static void check_2d(const Tensor& t, const char* what) {
    if (t.shape.size() != 2) throw FerriteError(FerriteError::InvalidArg, std::string(what) + " must be 2-d");
}

void HipBackend::matmul(const Tensor& x, const Tensor& w, const Tensor* bias, Tensor& out) {
    rec("matmul"); rec("matmul");   // the reference records this op twice (cpu.rs:89-90)
    check_2d(x, "matmul x"); check_2d(w, "matmul w");
    const size_t n = x.shape[0], k = x.shape[1], o = w.shape[0];
    if (k != w.shape[1]) throw FerriteError(FerriteError::ShapeMismatch, "matmul: x and w disagree on k");
    if (out.shape != std::vector<size_t>{n, o}) throw FerriteError(FerriteError::InvalidArg, "matmul out shape");
    if (bias && bias->numel() != o) throw FerriteError(FerriteError::InvalidArg, "matmul bias shape");
    DevBuf dx(n * k * 4), dw(o * k * 4), dout(n * o * 4), db(bias ? o * 4 : 0);
    dx.upload(x.data.data(), n * k * 4);
    dw.upload(w.data.data(), o * k * 4);
    if (bias) db.upload(bias->data.data(), o * 4);
    ck(api_->ferrite_matmul_f32(static_cast<const float*>(dx.ptr), static_cast<const float*>(dw.ptr),
                                bias ? static_cast<const float*>(db.ptr) : nullptr, static_cast<float*>(dout.ptr),
                                (int)n, (int)k, (int)o, stream_), "matmul");
    sync();
    dout.download(out.data.data(), n * o * 4);
}

void HipBackend::swiglu_limited(const Tensor& gate_up, float limit, Tensor& out) {
    rec("swiglu");
    check_2d(gate_up, "swiglu");
    const size_t n = gate_up.shape[0], two_i = gate_up.shape[1];
    if (two_i % 2) throw FerriteError(FerriteError::InvalidArg, "swiglu last dim must be even");
    if (out.shape != std::vector<size_t>{n, two_i / 2}) throw FerriteError(FerriteError::InvalidArg, "swiglu out shape");
    DevBuf dg(n * two_i * 4), dout(n * two_i * 2);
    dg.upload(gate_up.data.data(), n * two_i * 4);
    ck(api_->ferrite_swiglu_limited_f32(static_cast<const float*>(dg.ptr), limit, static_cast<float*>(dout.ptr), (int)n,
                                        (int)(two_i / 2), stream_), "swiglu");
    sync();
    dout.download(out.data.data(), n * two_i * 2);
}

// cpu.rs:124-143: the last dimension is normalised; w has that many elements; out has x's shape
void HipBackend::rmsnorm(const Tensor& x, const Tensor& w, float eps, Tensor& out) {
    rec("rmsnorm");
    if (x.shape.empty()) throw FerriteError(FerriteError::InvalidArg, "rmsnorm rank 0");
    const size_t dim = x.shape.back(), n = x.numel() / dim;
    if (w.numel() != dim || out.shape != x.shape) throw FerriteError(FerriteError::InvalidArg, "rmsnorm shape mismatch");
    DevBuf dx(n * dim * 4), dw(dim * 4), dout(n * dim * 4);
    dx.upload(x.data.data(), n * dim * 4);
    dw.upload(w.data.data(), dim * 4);
    ck(api_->ferrite_rmsnorm_f32(static_cast<const float*>(dx.ptr), static_cast<const float*>(dw.ptr), eps,
                                 static_cast<float*>(dout.ptr), (int)n, (int)dim, stream_), "rmsnorm");
    sync();
    dout.download(out.data.data(), n * dim * 4);
}

// cpu.rs:788-807: x [s,h], residual [s,nh,h], post [s,nh], comb [s,nh,nh] -> [s,nh,h]
Tensor HipBackend::hc_post(const Tensor& x, const Tensor& residual, const Tensor& post, const Tensor& comb) {
    rec("hc_post");
    check_2d(x, "hc_post x");
    if (residual.shape.size() != 3) throw FerriteError(FerriteError::InvalidArg, "hc_post residual must be [s,nh,h]");
    const size_t s = x.shape[0], h = x.shape[1], nh = residual.shape[1];
    if (residual.shape != std::vector<size_t>{s, nh, h} || post.shape != std::vector<size_t>{s, nh} ||
        comb.shape != std::vector<size_t>{s, nh, nh})
        throw FerriteError(FerriteError::ShapeMismatch, "hc_post shape mismatch");
    Tensor out = Tensor::zeros({s, nh, h});
    DevBuf dx(s * h * 4), dr(s * nh * h * 4), dp(s * nh * 4), dc(s * nh * nh * 4), dout(s * nh * h * 4);
    dx.upload(x.data.data(), s * h * 4);
    dr.upload(residual.data.data(), s * nh * h * 4);
    dp.upload(post.data.data(), s * nh * 4);
    dc.upload(comb.data.data(), s * nh * nh * 4);
    ck(api_->ferrite_hc_post_f32(static_cast<const float*>(dx.ptr), static_cast<const float*>(dr.ptr),
                                 static_cast<const float*>(dp.ptr), static_cast<const float*>(dc.ptr),
                                 static_cast<float*>(dout.ptr), (int)s, (int)nh, (int)h, stream_), "hc_post");
    sync();
    dout.download(out.data.data(), s * nh * h * 4);
    return out;
}

void HipBackend::moe_route(const Tensor& logits, const Tensor& bias, size_t topk, float routed_scaling, Tensor& probs,
                           Tensor& ids, int n_group, int topk_group) {
    rec("moe_route"); rec("moe_route");
    check_2d(logits, "logits");
    const size_t n = logits.shape[0], e = logits.shape[1];
    if (bias.numel() != e) throw FerriteError(FerriteError::InvalidArg, "router bias shape");
    if (probs.shape != std::vector<size_t>{n, topk} || ids.shape != std::vector<size_t>{n, topk})
        throw FerriteError(FerriteError::InvalidArg, "router out shape");
    DevBuf dl(n * e * 4), db(e * 4), dp(n * topk * 4), di(n * topk * 4);
    dl.upload(logits.data.data(), n * e * 4);
    db.upload(bias.data.data(), e * 4);
    ck(api_->ferrite_moe_route(static_cast<const float*>(dl.ptr), static_cast<const float*>(db.ptr), (int)n, (int)e,
                               (int)topk, n_group, topk_group, routed_scaling, static_cast<float*>(dp.ptr),
                               static_cast<float*>(di.ptr), nullptr, stream_), "moe_route");
    sync();
    dp.download(probs.data.data(), n * topk * 4);
    di.download(ids.data.data(), n * topk * 4);
}

void HipBackend::begin_capture() {
    recorded_.clear();
    ck(api_->ferrite_graph_begin(stream_), "graph_begin");
    capturing_ = true;
}

OpTrace HipBackend::end_capture() {
    capturing_ = false;
    OpTrace t;
    int rc = api_->ferrite_graph_end(stream_, &t.graph_exec);
    t.ops.swap(recorded_);
    if (rc != FERRITE_OK) throw std::logic_error(std::string("graph capture failed: ") + api_->ferrite_hip_last_error());
    return t;
}

void HipBackend::begin_verify(const OpTrace& trace) {
    if (!trace.graph_exec) throw FerriteError(FerriteError::InvalidArg, "trace holds no graph");
    verify_ok_ = api_->ferrite_graph_launch(trace.graph_exec, stream_) == FERRITE_OK;
}

bool HipBackend::end_verify() {
    return hipStreamSynchronize(static_cast<hipStream_t>(stream_)) == hipSuccess && verify_ok_;
}

void HipBackend::graph_destroy(OpTrace& trace) {
    if (trace.graph_exec) api_->ferrite_graph_destroy(trace.graph_exec);
    trace.graph_exec = nullptr;
}

MoeLayerDev HipBackend::load_moe_layer(const ferrite_moe_shape& s, const MoeHostWeights& w) {
    MoeLayerDev L;
    L.shape = s;
    const size_t E = s.n_experts, H = s.hidden, I = s.inter, Is = s.shared_inter;
    auto put = [&](const void* src, size_t bytes) -> const void* {
        if (!src || bytes == 0) return nullptr;
        L.storage.emplace_back(bytes);
        L.storage.back().upload(src, bytes);
        return L.storage.back().ptr;
    };
    L.dev.router_w = static_cast<const float*>(put(w.router_w, E * H * 4));
    L.dev.router_bias = static_cast<const float*>(put(w.router_bias, E * 4));
    L.dev.gate_w = static_cast<const uint8_t*>(put(w.gate_w, E * I * H / 2));
    L.dev.gate_s = static_cast<const uint8_t*>(put(w.gate_s, E * I * H / 32));
    L.dev.up_w = static_cast<const uint8_t*>(put(w.up_w, E * I * H / 2));
    L.dev.up_s = static_cast<const uint8_t*>(put(w.up_s, E * I * H / 32));
    L.dev.down_w = static_cast<const uint8_t*>(put(w.down_w, E * H * I / 2));
    L.dev.down_s = static_cast<const uint8_t*>(put(w.down_s, E * H * I / 32));
    L.dev.sh_gate_w = static_cast<const uint8_t*>(put(w.sh_gate_w, Is * H / 2));
    L.dev.sh_gate_s = static_cast<const uint8_t*>(put(w.sh_gate_s, Is * H / 32));
    L.dev.sh_up_w = static_cast<const uint8_t*>(put(w.sh_up_w, Is * H / 2));
    L.dev.sh_up_s = static_cast<const uint8_t*>(put(w.sh_up_s, Is * H / 32));
    L.dev.sh_down_w = static_cast<const uint8_t*>(put(w.sh_down_w, H * Is / 2));
    L.dev.sh_down_s = static_cast<const uint8_t*>(put(w.sh_down_s, H * Is / 32));
    const size_t pb = api_->ferrite_moe_packed_bytes(&L.shape);
    if (pb) {
        L.packed = DevBuf(pb);
        ck(api_->ferrite_moe_pack_weights(&L.shape, &L.dev, static_cast<uint8_t*>(L.packed.ptr), stream_), "pack_weights");
        sync();
    }
    return L;
}

void HipBackend::moe_layer_dev_mxfp4(MoeLayerDev& layer, const DevBuf& x, int x_dtype, int n, DevBuf& out,
                                     int out_dtype, int mode) {
    rec("moe_layer_mxfp4");
    if (n <= 0) throw FerriteError(FerriteError::InvalidArg, "n must be positive");
    const size_t esz_x = x_dtype == FERRITE_DT_F32 ? 4 : 2, esz_o = out_dtype == FERRITE_DT_F32 ? 4 : 2;
    if (x.bytes < (size_t)n * layer.shape.hidden * esz_x) throw FerriteError(FerriteError::ShapeMismatch, "x too small");
    if (out.bytes < (size_t)n * layer.shape.hidden * esz_o) throw FerriteError(FerriteError::InvalidArg, "out too small");
    // A mode that declines this call is not an error: the caller falls back (cuda.rs:5763-5765,5926-5937), two-term
    // MFMA -> one-term MFMA -> the f32 mode (the MFMA modes decline hidden / intermediate sizes that are not
    // multiples of 128; the f32 mode serves those from the checkpoint-layout weights).
    {
        const int chain[3] = {FERRITE_MODE_MFMA_FP8_X2, FERRITE_MODE_MFMA_FP8, FERRITE_MODE_F32_CHECK};
        int at = 0;
        while (at < 3 && chain[at] != mode) ++at;
        for (int i = at; i < 3; ++i) {
            const int rc = api_->ferrite_moe_layer_check(&layer.shape, n, chain[i]);
            if (rc == FERRITE_OK) { mode = chain[i]; break; }
            if (rc != FERRITE_DECLINED) break;
        }
    }
    if (layer.workspace_n != n || layer.workspace_mode != mode) {
        if (capturing_) throw FerriteError(FerriteError::InvalidArg, "workspace must be sized before capture");
        const size_t wb = api_->ferrite_moe_layer_workspace_bytes(&layer.shape, n, mode);
        if (wb == 0) throw FerriteError(FerriteError::InvalidArg, "unsupported shape / mode");
        layer.workspace = DevBuf(wb);
        ck(api_->ferrite_moe_layer_workspace_init(&layer.shape, n, mode, layer.workspace.ptr, wb, stream_), "workspace_init");
        layer.workspace_n = n;
        layer.workspace_mode = mode;
    }
    ck(api_->ferrite_moe_layer_mxfp4(&layer.shape, &layer.dev, static_cast<const uint8_t*>(layer.packed.ptr), x.ptr,
                                     x_dtype, n, out.ptr, out_dtype, mode, layer.workspace.ptr, layer.workspace.bytes,
                                     stream_), "moe_layer_mxfp4");
}

}  // namespace ferrite
