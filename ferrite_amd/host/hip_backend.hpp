// C++ host side of the MI355X backend for ferrite's MoE FFN path.
//
// The reference's host side is Rust: `trait KernelBackend` / `trait GraphCapable`
// (crates/ferrite-kernel/src/lib.rs:67-266, graph.rs:48-64) implemented by CpuBackend / CudaBackend, with
// `Tensor` = shape + dtype tag + row-major f32 storage (crates/ferrite-types/src/lib.rs:77-86) and errors as
// `FerriteError::{ShapeMismatch, InvalidArg, IndexOutOfBounds}` (:143-159).  This header mirrors that interface for
// the ops on the path, over libferrite_hip.so (dlopen, identity check, `ck()` error mapping: cuda.rs:411-425,
// 2061-2102).  Methods take pre-allocated outputs and return errors by exception; they never allocate inside a capture.
#pragma once
#include <cstddef>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/ferrite_hip.h"

namespace ferrite {

enum class DType { F32, Bf16, F16, Fp8E4m3 };

struct FerriteError : std::runtime_error {
    enum Kind { ShapeMismatch, InvalidArg, IndexOutOfBounds } kind;
    FerriteError(Kind k, const std::string& m) : std::runtime_error(m), kind(k) {}
};

// ferrite-types Tensor: f32 storage whatever the dtype tag says.
struct Tensor {
    std::vector<size_t> shape;
    DType dtype = DType::F32;
    std::vector<float> data;
    static Tensor zeros(std::vector<size_t> shape, DType dt = DType::F32);
    static Tensor from_f32(std::vector<size_t> shape, std::vector<float> v);
    size_t numel() const;
};

// graph.rs:20-45
struct OpRecord {
    std::string op;
    std::vector<std::vector<size_t>> shapes;
    bool operator==(const OpRecord& o) const { return op == o.op && shapes == o.shapes; }
};
struct OpTrace {
    std::vector<OpRecord> ops;
    void* graph_exec = nullptr;   // the instantiated hipGraph on a device backend
    size_t len() const { return ops.size(); }
};

// A device buffer owned by the backend's caller (the reference's DevBuf, cuda.rs:558-744, without the pool).
struct DevBuf {
    void* ptr = nullptr;
    size_t bytes = 0;
    DevBuf() = default;
    explicit DevBuf(size_t nbytes);
    ~DevBuf();
    DevBuf(const DevBuf&) = delete;
    DevBuf& operator=(const DevBuf&) = delete;
    DevBuf(DevBuf&& o) noexcept : ptr(o.ptr), bytes(o.bytes) { o.ptr = nullptr; o.bytes = 0; }
    DevBuf& operator=(DevBuf&& o) noexcept;
    void upload(const void* src, size_t nbytes);
    void download(void* dst, size_t nbytes) const;
};

// Host-side description of one layer's checkpoint-layout weights (pointers into caller memory).
struct MoeHostWeights {
    const float* router_w;
    const float* router_bias;   // may be null (zeros)
    const uint8_t *gate_w, *gate_s, *up_w, *up_s, *down_w, *down_s;
    const uint8_t *sh_gate_w, *sh_gate_s, *sh_up_w, *sh_up_s, *sh_down_w, *sh_down_s;
};

struct MoeLayerDev {
    ferrite_moe_shape shape{};
    ferrite_moe_weights dev{};          // device pointers (checkpoint layout)
    std::vector<DevBuf> storage;
    DevBuf packed;                       // tile layout for the MFMA path (empty when the shape is declined)
    DevBuf workspace;
    int workspace_n = 0, workspace_mode = -1;
};

class HipBackend {
  public:
    explicit HipBackend(const std::string& so_path, int device = 0);
    ~HipBackend();
    HipBackend(const HipBackend&) = delete;

    std::string build_id() const;

    // ---- KernelBackend, the ops on the path (host tensors in, pre-allocated host tensors out) ----
    void matmul(const Tensor& x, const Tensor& w, const Tensor* bias, Tensor& out);                  // lib.rs:73
    void swiglu_limited(const Tensor& gate_up, float limit, Tensor& out);                            // lib.rs:83-85
    void rmsnorm(const Tensor& x, const Tensor& w, float eps, Tensor& out);                          // lib.rs:76
    Tensor hc_post(const Tensor& x, const Tensor& residual, const Tensor& post, const Tensor& comb); // lib.rs:256
    void moe_route(const Tensor& logits, const Tensor& bias, size_t topk, float routed_scaling, Tensor& probs,
                   Tensor& ids, int n_group = 1, int topk_group = 1);                                // lib.rs:194-206

    // ---- GraphCapable (graph.rs:48-64 with the device semantics of cuda.rs:3043-3092) ----
    void begin_capture();
    OpTrace end_capture();
    void begin_verify(const OpTrace& trace);
    bool end_verify();
    void graph_destroy(OpTrace& trace);

    // ---- inherent device chain: the counterpart of CudaBackend::moe_layer_dev (cuda.rs:5604-6142) ----
    MoeLayerDev load_moe_layer(const ferrite_moe_shape& shape, const MoeHostWeights& w);
    // x / out: device buffers holding [n, hidden] in x_dtype / out_dtype (FERRITE_DT_*).  Sizes the layer's
    // workspace on first use for (n, mode): call once before capturing.
    void moe_layer_dev_mxfp4(MoeLayerDev& layer, const DevBuf& x, int x_dtype, int n, DevBuf& out, int out_dtype,
                             int mode);
    void sync();

  private:
    struct Api;
    std::unique_ptr<Api> api_;
    void* so_ = nullptr;
    void* stream_ = nullptr;
    bool capturing_ = false;
    bool verify_ok_ = false;
    std::vector<OpRecord> recorded_;
    void ck(int rc, const char* what) const;
    void rec(const char* op);
};

}  // namespace ferrite
