// Checkpoint -> device for one MoE layer: a safetensors header reader and a streaming loader that stages the
// layer's expert tensors one expert at a time and has the device repack them into the tile order the MFMA kernels
// stream.  Nothing is dequantised on the way ("loading never dequantises", crates/ferrite-models/src/dsv41/
// weights.rs:12-16); a checkpoint whose experts are unquantised is quantised to MXFP4 on the device.
//
// The reference's counterparts: `TensorView` / `SafetensorsIndex::{read_header, validate}`
// (crates/ferrite-models/src/dsv41/weights.rs:814-905), the tensor names of one layer's MoE
// (weights.rs:333-354 for DeepSeek-V4.1, crates/ferrite-model/src/weights.rs:133-149 for GLM), and the scale-row
// pitch rule `sf_plane_pitch` (weights.rs:599) with the story behind it in
// kernels/cuda/dsv41_experts_mxf4.cu:121-168.
#pragma once
#include <cstddef>
#include <cstdint>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/ferrite_hip.h"
#include "hip_backend.hpp"

namespace ferrite {

// A byte-range view into a safetensors file (weights.rs:814-823); offsets are relative to the data section.
struct TensorView {
    std::string dtype;
    std::vector<size_t> shape;
    uint64_t begin = 0, end = 0;
    size_t numel() const;
};

// One tensor the loader expects (weights.rs:53-58, without the sharding rule: one GPU holds the layer).
struct TensorSpec {
    std::string name;
    std::vector<size_t> shape;
};

// weights.rs:825-905.  Errors are FerriteError::InvalidArg with the reference's wording ("open <path>: ...",
// "header len: ...", "implausible header length N", "header json: ...", "safetensors header is not an object").
class SafetensorsIndex {
  public:
    static SafetensorsIndex read_header(const std::string& path);
    static SafetensorsIndex parse_header(const char* json, size_t len);
    // Names that are missing, and "name: shape [..] != [..]" for a wrong shape (weights.rs:882-905).
    std::vector<std::string> validate(const std::vector<TensorSpec>& specs) const;
    const TensorView* find(const std::string& name) const;

    std::unordered_map<std::string, TensorView> tensors;
    uint64_t data_start = 0;   // 8 + header length: where the data section begins in the file
};

// A read-only mapping of a checkpoint shard.
class MappedFile {
  public:
    explicit MappedFile(const std::string& path);
    ~MappedFile();
    MappedFile(const MappedFile&) = delete;
    MappedFile& operator=(const MappedFile&) = delete;
    const uint8_t* data() const { return data_; }
    size_t size() const { return size_; }

  private:
    const uint8_t* data_ = nullptr;
    size_t size_ = 0;
};

// Which checkpoint family names the layer's tensors.
//   Dsv41: "<prefix>.gate.weight" [E,H], "<prefix>.gate.bias" [E], "<prefix>.experts.<e>.w1|w2|w3.weight" I8
//          [out, in/2] + ".scale" F8_E8M0 [out, in/32] (w1 gate, w3 up, w2 down), "<prefix>.shared_experts.w*"
//          with prefix = "layers.<L>.ffn".
//   Glm:   "<prefix>.gate.weight", "<prefix>.gate.e_score_correction_bias", "<prefix>.experts.<e>.gate_proj|
//          up_proj|down_proj.weight" [out, in] BF16 or F32, "<prefix>.shared_expert.*_proj.weight"; these are
//          quantised to MXFP4 on the device (quant.rs:217-238, block 32, power-of-two scale).
enum class MoeNaming { Dsv41 = 0, Glm = 1 };

// The tensors of one layer's MoE with their on-disk shapes.  An fp4 expert weight is described packed
// ([out, in/2]) and its scale as one byte per (row, 32 columns) (weights.rs:889-894).
std::vector<TensorSpec> moe_layer_specs(MoeNaming naming, const std::string& prefix, const ferrite_moe_shape& shape);

// The physical row stride of an e8m0 scale plane whose rows hold `cols` bytes, for loaders that keep planes in
// the checkpoint layout on the device: rows padded to the next multiple of 16 bytes (weights.rs:599).
inline size_t sf_plane_pitch(size_t cols) { return (cols + 15) & ~size_t(15); }

// One shard of a checkpoint that is split over several files (both pointers borrowed).
struct CheckpointShard {
    const MappedFile* file;
    const SafetensorsIndex* index;
};

struct LoadStats {
    uint64_t source_bytes = 0;   // bytes of the layer's tensors read from the file
    uint64_t packed_bytes = 0;   // size of the packed buffer
    double seconds = 0.0;        // wall time of the whole load, device work included
    int workers = 0;
};

struct LoadOptions {
    int workers = 8;             // staging threads, each with its own pinned buffer, device buffer and stream
    bool pad_scale_rows = false; // stage scale planes with sf_plane_pitch rows (exercises the pitch argument)
};

// Streams one layer from a mapped checkpoint into `packed_dev` (ferrite_moe_packed_bytes(shape) bytes of device
// memory) and `router_bias_dev` ([E] f32, may be null when the checkpoint has no bias tensor: an absent bias
// leaves it untouched).  Every tensor is validated (name, dtype, shape, byte range inside the file) before any
// byte moves; a failure throws FerriteError and leaves the device buffers unspecified.
class MoeCheckpointLoader {
  public:
    explicit MoeCheckpointLoader(const std::string& hip_so_path, int device = 0);
    ~MoeCheckpointLoader();
    MoeCheckpointLoader(const MoeCheckpointLoader&) = delete;

    size_t packed_bytes(const ferrite_moe_shape& shape) const;
    LoadStats load_layer(const MappedFile& file, const SafetensorsIndex& index, MoeNaming naming,
                         const std::string& prefix, const ferrite_moe_shape& shape, uint8_t* packed_dev,
                         float* router_bias_dev, const LoadOptions& opt = LoadOptions()) const;
    // The same over a checkpoint split into shards: every tensor is taken from the first shard that names it (a
    // layer's experts usually straddle two or three files of a released checkpoint).
    LoadStats load_layer(const std::vector<CheckpointShard>& shards, MoeNaming naming, const std::string& prefix,
                         const ferrite_moe_shape& shape, uint8_t* packed_dev, float* router_bias_dev,
                         const LoadOptions& opt = LoadOptions()) const;

  private:
    struct Api;
    struct Slot {              // one staging worker's resources; every buffer is two halves used in turn
        uint8_t* pinned = nullptr;
        uint8_t* dev = nullptr;
        uint8_t* qdev = nullptr;   // output of the device quantiser (unquantised checkpoints only)
        size_t bytes = 0, qbytes = 0;   // size of one half
        void* stream = nullptr;
        void* done[2] = {nullptr, nullptr};   // recorded after the pack kernels that read a half
    };
    void ensure_slots(int count, size_t bytes, size_t qbytes) const;
    static void release(Slot& sl);
    Api* api_;
    void* so_ = nullptr;
    int device_ = 0;
    mutable std::vector<Slot> slots_;
    mutable std::mutex mu_;     // one load at a time per loader: the slots are shared state
};

}  // namespace ferrite
