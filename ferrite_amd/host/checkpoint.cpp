#include "checkpoint.hpp"

#include <dlfcn.h>
#include <fcntl.h>
#include <hip/hip_runtime_api.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <cerrno>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <exception>
#include <mutex>
#include <thread>

namespace ferrite {

namespace {

[[noreturn]] void config_error(const std::string& m) { throw FerriteError(FerriteError::InvalidArg, m); }

void hipck(hipError_t e, const char* what) {
    if (e != hipSuccess) config_error(std::string("HIP ") + what + ": " + hipGetErrorString(e));
}

// ---- a JSON reader for the safetensors header: objects, arrays, strings, numbers, true/false/null ----------
struct Json {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    double num = 0.0;
    bool is_uint = false;
    uint64_t uint = 0;
    std::string str;
    std::vector<Json> items;                              // Array
    std::vector<std::pair<std::string, Json>> members;    // Object, in file order
    const Json* get(const char* key) const {
        if (kind != Object) return nullptr;
        for (const auto& m : members)
            if (m.first == key) return &m.second;
        return nullptr;
    }
};

class JsonParser {
  public:
    JsonParser(const char* p, size_t n) : p_(p), end_(p + n) {}
    Json parse_document() {
        Json v = value(0);
        ws();
        if (p_ != end_) fail("trailing characters");
        return v;
    }

  private:
    const char* p_;
    const char* end_;
    [[noreturn]] void fail(const char* what) const { config_error(std::string("header json: ") + what); }
    void ws() {
        while (p_ != end_ && (*p_ == ' ' || *p_ == '\t' || *p_ == '\n' || *p_ == '\r')) ++p_;
    }
    bool lit(const char* s) {
        const size_t n = strlen(s);
        if ((size_t)(end_ - p_) < n || memcmp(p_, s, n) != 0) return false;
        p_ += n;
        return true;
    }
    static void put_utf8(std::string& out, uint32_t c) {
        if (c < 0x80) out += (char)c;
        else if (c < 0x800) { out += (char)(0xC0 | (c >> 6)); out += (char)(0x80 | (c & 0x3F)); }
        else if (c < 0x10000) {
            out += (char)(0xE0 | (c >> 12)); out += (char)(0x80 | ((c >> 6) & 0x3F)); out += (char)(0x80 | (c & 0x3F));
        } else {
            out += (char)(0xF0 | (c >> 18)); out += (char)(0x80 | ((c >> 12) & 0x3F));
            out += (char)(0x80 | ((c >> 6) & 0x3F)); out += (char)(0x80 | (c & 0x3F));
        }
    }
    uint32_t hex4() {
        if (end_ - p_ < 4) fail("short \\u escape");
        uint32_t v = 0;
        for (int i = 0; i < 4; ++i) {
            const char c = *p_++;
            v <<= 4;
            if (c >= '0' && c <= '9') v |= (uint32_t)(c - '0');
            else if (c >= 'a' && c <= 'f') v |= (uint32_t)(c - 'a' + 10);
            else if (c >= 'A' && c <= 'F') v |= (uint32_t)(c - 'A' + 10);
            else fail("bad \\u escape");
        }
        return v;
    }
    std::string string() {
        if (p_ == end_ || *p_ != '"') fail("expected a string");
        ++p_;
        std::string out;
        for (;;) {
            if (p_ == end_) fail("unterminated string");
            const unsigned char c = (unsigned char)*p_++;
            if (c == '"') return out;
            if (c < 0x20) fail("control character in string");
            if (c != '\\') { out += (char)c; continue; }
            if (p_ == end_) fail("unterminated escape");
            const char e = *p_++;
            switch (e) {
                case '"': out += '"'; break;
                case '\\': out += '\\'; break;
                case '/': out += '/'; break;
                case 'b': out += '\b'; break;
                case 'f': out += '\f'; break;
                case 'n': out += '\n'; break;
                case 'r': out += '\r'; break;
                case 't': out += '\t'; break;
                case 'u': {
                    uint32_t c1 = hex4();
                    if (c1 >= 0xD800 && c1 < 0xDC00) {   // surrogate pair
                        if (end_ - p_ < 2 || p_[0] != '\\' || p_[1] != 'u') fail("lone surrogate");
                        p_ += 2;
                        const uint32_t c2 = hex4();
                        if (c2 < 0xDC00 || c2 > 0xDFFF) fail("bad surrogate pair");
                        c1 = 0x10000 + ((c1 - 0xD800) << 10) + (c2 - 0xDC00);
                    }
                    put_utf8(out, c1);
                    break;
                }
                default: fail("bad escape");
            }
        }
    }
    Json number() {
        const char* s = p_;
        if (p_ != end_ && *p_ == '-') ++p_;
        bool integer = true;
        while (p_ != end_ && ((*p_ >= '0' && *p_ <= '9') || *p_ == '.' || *p_ == 'e' || *p_ == 'E' || *p_ == '+' ||
                              *p_ == '-')) {
            if (*p_ < '0' || *p_ > '9') integer = false;
            ++p_;
        }
        if (p_ == s || (p_ - s == 1 && *s == '-')) fail("bad number");
        Json v;
        v.kind = Json::Number;
        const std::string t(s, p_);
        v.num = strtod(t.c_str(), nullptr);
        if (integer && *s != '-' && t.size() <= 19) {
            v.is_uint = true;
            v.uint = strtoull(t.c_str(), nullptr, 10);
        }
        return v;
    }
    Json value(int depth) {
        if (depth > 64) fail("nesting too deep");
        ws();
        if (p_ == end_) fail("unexpected end");
        Json v;
        const char c = *p_;
        if (c == '{') {
            ++p_;
            v.kind = Json::Object;
            ws();
            if (p_ != end_ && *p_ == '}') { ++p_; return v; }
            for (;;) {
                ws();
                std::string key = string();
                ws();
                if (p_ == end_ || *p_ != ':') fail("expected ':'");
                ++p_;
                v.members.emplace_back(std::move(key), value(depth + 1));
                ws();
                if (p_ == end_) fail("unterminated object");
                if (*p_ == ',') { ++p_; continue; }
                if (*p_ == '}') { ++p_; return v; }
                fail("expected ',' or '}'");
            }
        }
        if (c == '[') {
            ++p_;
            v.kind = Json::Array;
            ws();
            if (p_ != end_ && *p_ == ']') { ++p_; return v; }
            for (;;) {
                v.items.push_back(value(depth + 1));
                ws();
                if (p_ == end_) fail("unterminated array");
                if (*p_ == ',') { ++p_; continue; }
                if (*p_ == ']') { ++p_; return v; }
                fail("expected ',' or ']'");
            }
        }
        if (c == '"') { v.kind = Json::String; v.str = string(); return v; }
        if (lit("true")) { v.kind = Json::Bool; v.num = 1; return v; }
        if (lit("false")) { v.kind = Json::Bool; return v; }
        if (lit("null")) return v;
        return number();
    }
};

std::string shape_str(const std::vector<size_t>& s) {
    std::string o = "[";
    for (size_t i = 0; i < s.size(); ++i) o += (i ? ", " : "") + std::to_string(s[i]);
    return o + "]";
}

size_t dtype_size(const std::string& dt) {
    if (dt == "I8" || dt == "U8" || dt == "F8_E8M0" || dt == "F8_E4M3" || dt == "F8_E5M2" || dt == "BOOL") return 1;
    if (dt == "BF16" || dt == "F16" || dt == "I16" || dt == "U16") return 2;
    if (dt == "F32" || dt == "I32" || dt == "U32") return 4;
    if (dt == "F64" || dt == "I64" || dt == "U64") return 8;
    return 0;
}

}  // namespace

size_t TensorView::numel() const {
    size_t n = 1;
    for (size_t d : shape) n *= d;
    return n;
}

SafetensorsIndex SafetensorsIndex::parse_header(const char* json, size_t len) {
    const Json doc = JsonParser(json, len).parse_document();
    if (doc.kind != Json::Object) config_error("safetensors header is not an object");
    SafetensorsIndex idx;
    for (const auto& m : doc.members) {
        if (m.first == "__metadata__") continue;
        TensorView v;
        // the reference is lenient here (missing fields read as empty, weights.rs:856-875); so is this reader
        if (const Json* d = m.second.get("dtype"); d && d->kind == Json::String) v.dtype = d->str;
        if (const Json* s = m.second.get("shape"); s && s->kind == Json::Array)
            for (const Json& e : s->items)
                if (e.kind == Json::Number && e.is_uint) v.shape.push_back((size_t)e.uint);
        if (const Json* o = m.second.get("data_offsets"); o && o->kind == Json::Array && o->items.size() == 2) {
            v.begin = o->items[0].is_uint ? o->items[0].uint : 0;
            v.end = o->items[1].is_uint ? o->items[1].uint : 0;
        }
        idx.tensors.emplace(m.first, std::move(v));
    }
    return idx;
}

SafetensorsIndex SafetensorsIndex::read_header(const std::string& path) {
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) config_error("open " + path + ": " + strerror(errno));
    unsigned char len8[8];
    if (fread(len8, 1, 8, f) != 8) {
        fclose(f);
        config_error("header len: failed to fill whole buffer");
    }
    uint64_t hlen = 0;
    for (int i = 7; i >= 0; --i) hlen = (hlen << 8) | len8[i];
    if (hlen > 100ull * 1024 * 1024) {
        fclose(f);
        config_error("implausible header length " + std::to_string(hlen));
    }
    std::string buf((size_t)hlen, '\0');
    if (hlen && fread(&buf[0], 1, (size_t)hlen, f) != hlen) {
        fclose(f);
        config_error("header body: failed to fill whole buffer");
    }
    fclose(f);
    SafetensorsIndex idx = parse_header(buf.data(), buf.size());
    idx.data_start = 8 + hlen;
    return idx;
}

const TensorView* SafetensorsIndex::find(const std::string& name) const {
    auto it = tensors.find(name);
    return it == tensors.end() ? nullptr : &it->second;
}

std::vector<std::string> SafetensorsIndex::validate(const std::vector<TensorSpec>& specs) const {
    std::vector<std::string> missing;
    for (const TensorSpec& s : specs) {
        const TensorView* v = find(s.name);
        if (!v) missing.push_back(s.name);
        else if (v->shape != s.shape) missing.push_back(s.name + ": shape " + shape_str(v->shape) + " != " + shape_str(s.shape));
    }
    return missing;
}

MappedFile::MappedFile(const std::string& path) {
    const int fd = open(path.c_str(), O_RDONLY);
    if (fd < 0) config_error("open " + path + ": " + strerror(errno));
    struct stat st;
    if (fstat(fd, &st) != 0) {
        close(fd);
        config_error("stat " + path + ": " + strerror(errno));
    }
    size_ = (size_t)st.st_size;
    if (size_) {
        void* p = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd, 0);
        if (p == MAP_FAILED) {
            close(fd);
            config_error("mmap " + path + ": " + strerror(errno));
        }
        data_ = static_cast<const uint8_t*>(p);
    }
    close(fd);
}
MappedFile::~MappedFile() {
    if (data_) munmap(const_cast<uint8_t*>(data_), size_);
}

// ---- names ----------------------------------------------------------------------------------------------------
namespace {
struct MatNames { const char* gate; const char* up; const char* down; };
MatNames mat_names(MoeNaming n) {
    return n == MoeNaming::Dsv41 ? MatNames{"w1", "w3", "w2"} : MatNames{"gate_proj", "up_proj", "down_proj"};
}
std::string expert_prefix(MoeNaming n, const std::string& prefix, int e, int n_experts) {
    if (e == n_experts) return prefix + (n == MoeNaming::Dsv41 ? ".shared_experts" : ".shared_expert");
    return prefix + ".experts." + std::to_string(e);
}
std::string bias_name(MoeNaming n, const std::string& prefix) {
    return prefix + (n == MoeNaming::Dsv41 ? ".gate.bias" : ".gate.e_score_correction_bias");
}
}  // namespace

std::vector<TensorSpec> moe_layer_specs(MoeNaming naming, const std::string& prefix, const ferrite_moe_shape& s) {
    std::vector<TensorSpec> out;
    const size_t H = s.hidden, E = s.n_experts;
    out.push_back({prefix + ".gate.weight", {E, H}});
    out.push_back({bias_name(naming, prefix), {E}});
    const MatNames mn = mat_names(naming);
    for (int e = 0; e <= s.n_experts; ++e) {
        if (e == s.n_experts && s.shared_inter == 0) break;
        const size_t I = e == s.n_experts ? s.shared_inter : s.inter;
        const std::string p = expert_prefix(naming, prefix, e, s.n_experts);
        const struct { const char* n; size_t o, k; } mats[3] = {{mn.gate, I, H}, {mn.down, H, I}, {mn.up, I, H}};
        for (const auto& m : mats) {
            if (naming == MoeNaming::Dsv41) {
                out.push_back({p + "." + m.n + ".weight", {m.o, m.k / 2}});
                out.push_back({p + "." + m.n + ".scale", {m.o, m.k / 32}});
            } else {
                out.push_back({p + "." + m.n + ".weight", {m.o, m.k}});
            }
        }
    }
    return out;
}

// ---- the loader -----------------------------------------------------------------------------------------------
struct MoeCheckpointLoader::Api {
#define FN(name) decltype(&::name) name = nullptr
    FN(ferrite_kernel_abi_version); FN(ferrite_hip_last_error); FN(ferrite_moe_packed_bytes);
    FN(ferrite_moe_pack_expert); FN(ferrite_moe_pack_router); FN(ferrite_mxfp4_quant);
#undef FN
};

MoeCheckpointLoader::MoeCheckpointLoader(const std::string& so_path, int device) : api_(new Api), device_(device) {
    so_ = dlopen(so_path.c_str(), RTLD_NOW | RTLD_LOCAL);
    if (!so_) {
        delete api_;
        config_error(std::string("dlopen ") + so_path + ": " + dlerror());
    }
#define LOAD(name)                                                                              \
    api_->name = reinterpret_cast<decltype(api_->name)>(dlsym(so_, #name));                      \
    if (!api_->name) { dlclose(so_); delete api_; config_error("missing symbol " #name); }
    LOAD(ferrite_kernel_abi_version); LOAD(ferrite_hip_last_error); LOAD(ferrite_moe_packed_bytes);
    LOAD(ferrite_moe_pack_expert); LOAD(ferrite_moe_pack_router); LOAD(ferrite_mxfp4_quant);
#undef LOAD
    if (api_->ferrite_kernel_abi_version() != FERRITE_ABI_VERSION) {
        dlclose(so_);
        delete api_;
        config_error("libferrite_hip.so ABI version mismatch");
    }
}

MoeCheckpointLoader::~MoeCheckpointLoader() {
    for (Slot& sl : slots_) release(sl);
    if (so_) dlclose(so_);
    delete api_;
}

void MoeCheckpointLoader::release(Slot& sl) {
    if (sl.stream) { (void)hipStreamSynchronize(static_cast<hipStream_t>(sl.stream)); (void)hipStreamDestroy(static_cast<hipStream_t>(sl.stream)); }
    for (void* ev : sl.done)
        if (ev) (void)hipEventDestroy(static_cast<hipEvent_t>(ev));
    if (sl.qdev) (void)hipFree(sl.qdev);
    if (sl.dev) (void)hipFree(sl.dev);
    if (sl.pinned) (void)hipHostFree(sl.pinned);
    sl = Slot{};
}

// Staging resources live as long as the loader: a model has many layers and each load reuses them.
void MoeCheckpointLoader::ensure_slots(int count, size_t bytes, size_t qbytes) const {
    if ((int)slots_.size() < count) slots_.resize((size_t)count);
    for (int i = 0; i < count; ++i) {
        Slot& sl = slots_[(size_t)i];
        if (!sl.stream) {
            hipStream_t st = nullptr;
            hipck(hipStreamCreateWithFlags(&st, hipStreamNonBlocking), "hipStreamCreate");   // default priority
            sl.stream = st;
        }
        for (void*& ev : sl.done)
            if (!ev) {
                hipEvent_t e = nullptr;
                hipck(hipEventCreateWithFlags(&e, hipEventDisableTiming), "hipEventCreate");
                ev = e;
            }
        if (sl.bytes < bytes) {   // two halves of `bytes` each
            if (sl.dev) (void)hipFree(sl.dev);
            if (sl.pinned) (void)hipHostFree(sl.pinned);
            sl.dev = sl.pinned = nullptr;
            sl.bytes = 0;
            hipck(hipHostMalloc(reinterpret_cast<void**>(&sl.pinned), 2 * bytes, hipHostMallocDefault), "hipHostMalloc");
            hipck(hipMalloc(reinterpret_cast<void**>(&sl.dev), 2 * bytes), "hipMalloc");
            sl.bytes = bytes;
        }
        if (sl.qbytes < qbytes) {
            if (sl.qdev) (void)hipFree(sl.qdev);
            sl.qdev = nullptr;
            sl.qbytes = 0;
            hipck(hipMalloc(reinterpret_cast<void**>(&sl.qdev), 2 * qbytes), "hipMalloc");
            sl.qbytes = qbytes;
        }
    }
}

size_t MoeCheckpointLoader::packed_bytes(const ferrite_moe_shape& shape) const {
    return api_->ferrite_moe_packed_bytes(&shape);
}

namespace {

// One matrix of one expert as the file holds it.
struct MatSrc {
    const uint8_t* w = nullptr;   // codes (Dsv41) or values (Glm)
    const uint8_t* s = nullptr;   // scales (Dsv41)
    size_t rows = 0, cols = 0;    // logical [out, in]
    size_t w_bytes = 0, esize = 0;
};

struct ExpertSrc { MatSrc gate, up, down; };

// The shard of a set that holds `name` (the first one that does), or null.
const CheckpointShard* shard_of(const std::vector<CheckpointShard>& shards, const std::string& name) {
    for (const CheckpointShard& sh : shards)
        if (sh.index->find(name)) return &sh;
    return nullptr;
}

const uint8_t* tensor_bytes(const std::vector<CheckpointShard>& shards, const std::string& name,
                            const std::vector<std::string>& dtypes, const std::vector<size_t>& shape, size_t* esize) {
    const CheckpointShard* sh = shard_of(shards, name);
    if (!sh) config_error("missing tensor " + name);
    const MappedFile& f = *sh->file;
    const SafetensorsIndex& idx = *sh->index;
    const TensorView* v = idx.find(name);
    bool dt_ok = false;
    for (const auto& d : dtypes) dt_ok = dt_ok || d == v->dtype;
    if (!dt_ok) config_error(name + ": dtype " + v->dtype + " is not one this path loads");
    if (v->shape != shape) config_error(name + ": shape " + shape_str(v->shape) + " != " + shape_str(shape));
    const size_t es = dtype_size(v->dtype);
    if (v->end < v->begin || v->end - v->begin != (uint64_t)v->numel() * es)
        config_error(name + ": data_offsets do not match shape and dtype");
    if (idx.data_start + v->end > f.size()) config_error(name + ": data runs past the end of the file");
    if (esize) *esize = es;
    return f.data() + idx.data_start + v->begin;
}

size_t align16(size_t v) { return (v + 15) & ~size_t(15); }
size_t align256(size_t v) { return (v + 255) & ~size_t(255); }

// Copies a scale plane [rows, cols] into rows of `pitch` bytes.
void copy_plane(uint8_t* dst, const uint8_t* src, size_t rows, size_t cols, size_t pitch) {
    if (pitch == cols) { memcpy(dst, src, rows * cols); return; }
    for (size_t r = 0; r < rows; ++r) memcpy(dst + r * pitch, src + r * cols, cols);
}

}  // namespace

LoadStats MoeCheckpointLoader::load_layer(const MappedFile& file, const SafetensorsIndex& index, MoeNaming naming,
                                          const std::string& prefix, const ferrite_moe_shape& s, uint8_t* packed_dev,
                                          float* router_bias_dev, const LoadOptions& opt) const {
    return load_layer(std::vector<CheckpointShard>{CheckpointShard{&file, &index}}, naming, prefix, s, packed_dev,
                      router_bias_dev, opt);
}

LoadStats MoeCheckpointLoader::load_layer(const std::vector<CheckpointShard>& shards, MoeNaming naming,
                                          const std::string& prefix, const ferrite_moe_shape& s, uint8_t* packed_dev,
                                          float* router_bias_dev, const LoadOptions& opt) const {
    if (shards.empty()) config_error("no checkpoint shard given");
    for (const CheckpointShard& sh : shards)
        if (!sh.file || !sh.index) config_error("null checkpoint shard");
    const auto t0 = std::chrono::steady_clock::now();
    if (!packed_dev) config_error("packed_dev is null");
    const size_t pbytes = api_->ferrite_moe_packed_bytes(&s);
    if (pbytes == 0) config_error("shape not supported by the MFMA path (hidden, inter, shared_inter multiples of 128)");
    const size_t H = s.hidden, E = s.n_experts;
    const bool quantised = naming == MoeNaming::Dsv41;
    const MatNames mn = mat_names(naming);
    const std::vector<std::string> code_dt = {"I8", "U8"}, scale_dt = {"F8_E8M0", "U8"}, val_dt = {"BF16", "F32"};

    // ---- resolve and validate everything first ----
    LoadStats stats;
    stats.packed_bytes = pbytes;
    size_t router_es = 0;
    const uint8_t* router_src = tensor_bytes(shards, prefix + ".gate.weight", val_dt, {E, H}, &router_es);
    stats.source_bytes += E * H * router_es;
    const uint8_t* bias_src = nullptr;
    size_t bias_es = 0;
    if (shard_of(shards, bias_name(naming, prefix))) {
        bias_src = tensor_bytes(shards, bias_name(naming, prefix), val_dt, {E}, &bias_es);
        stats.source_bytes += E * bias_es;
        if (!router_bias_dev) config_error("the checkpoint has a routing bias but router_bias_dev is null");
    }
    const int n_src = s.n_experts + (s.shared_inter > 0 ? 1 : 0);
    std::vector<ExpertSrc> experts((size_t)n_src);
    size_t slot_bytes = 0;
    for (int e = 0; e < n_src; ++e) {
        const size_t I = e == s.n_experts ? s.shared_inter : s.inter;
        const std::string p = expert_prefix(naming, prefix, e, s.n_experts);
        if (quantised && e == s.n_experts) {
            const CheckpointShard* sh = shard_of(shards, p + "." + mn.gate + ".weight");
            const TensorView* v = sh ? sh->index->find(p + "." + mn.gate + ".weight") : nullptr;
            if (v && v->dtype == "F8_E4M3")
                config_error(p + ": the shared expert is stored as F8_E4M3, which is not an MXFP4 tensor; load the layer "
                             "with shared_inter = 0 and run the shared expert on its own path");
        }
        auto resolve = [&](const char* nm, size_t o, size_t k) {
            MatSrc m;
            m.rows = o; m.cols = k;
            if (quantised) {
                m.w = tensor_bytes(shards, p + "." + nm + ".weight", code_dt, {o, k / 2}, nullptr);
                m.s = tensor_bytes(shards, p + "." + nm + ".scale", scale_dt, {o, k / 32}, nullptr);
                m.w_bytes = o * k / 2;
                m.esize = 1;
                stats.source_bytes += m.w_bytes + o * k / 32;
            } else {
                m.w = tensor_bytes(shards, p + "." + nm + ".weight", val_dt, {o, k}, &m.esize);
                m.w_bytes = o * k * m.esize;
                stats.source_bytes += m.w_bytes;
            }
            return m;
        };
        experts[e].gate = resolve(mn.gate, I, H);
        experts[e].up = resolve(mn.up, I, H);
        experts[e].down = resolve(mn.down, H, I);
        if (!quantised && (experts[e].gate.esize != experts[e].up.esize || experts[e].gate.esize != experts[e].down.esize))
            config_error(p + ": gate, up and down must share a dtype");
        // staged bytes of this expert: the three value/code matrices, the three scale planes at their staged pitch
        const size_t gu_pitch = opt.pad_scale_rows ? sf_plane_pitch(H / 32) : H / 32;
        const size_t dn_pitch = opt.pad_scale_rows ? sf_plane_pitch(I / 32) : I / 32;
        size_t need = 3 * align256(experts[e].gate.w_bytes);   // gate/up/down hold the same element count
        need += 2 * align256(I * gu_pitch) + align256(H * dn_pitch);
        if (need > slot_bytes) slot_bytes = need;
    }

    hipck(hipSetDevice(device_), "hipSetDevice");

    // ---- router and bias: small, converted to f32 on the host when stored as bf16; runs on the calling thread
    //      while the workers stream the experts ----
    auto load_router = [&]() {
        std::vector<float> rw(E * H), rb;
        auto to_f32 = [](const uint8_t* src, size_t es, size_t n, float* dst) {
            if (es == 4) { memcpy(dst, src, n * 4); return; }
            for (size_t i = 0; i < n; ++i) {
                uint16_t h;
                memcpy(&h, src + 2 * i, 2);
                const uint32_t u = (uint32_t)h << 16;
                memcpy(dst + i, &u, 4);
            }
        };
        to_f32(router_src, router_es, E * H, rw.data());
        DevBuf drw(E * H * 4);
        drw.upload(rw.data(), E * H * 4);
        const int rc = api_->ferrite_moe_pack_router(&s, static_cast<const float*>(drw.ptr), packed_dev, nullptr);
        if (rc) config_error(std::string("pack_router: rc=") + std::to_string(rc) + " " + api_->ferrite_hip_last_error());
        if (bias_src) {
            rb.resize(E);
            to_f32(bias_src, bias_es, E, rb.data());
            hipck(hipMemcpy(router_bias_dev, rb.data(), E * 4, hipMemcpyHostToDevice), "hipMemcpy bias");
        }
        hipck(hipStreamSynchronize(nullptr), "hipStreamSynchronize");   // drw is freed on return
    };

    // ---- experts: worker w stages experts w, w + W, ... through its own pinned buffer, device buffer and stream ----
    const int W = std::max(1, std::min(opt.workers, n_src));
    stats.workers = W;
    std::atomic<bool> failed{false};
    std::mutex err_mu;
    std::string err;
    size_t qbytes = 0;
    if (!quantised) {
        // room for the codes and scales the device quantiser writes (largest expert)
        for (int e = 0; e < n_src; ++e) {
            const size_t I = e == s.n_experts ? s.shared_inter : s.inter;
            qbytes = std::max(qbytes, 3 * align256(I * H / 2) + 3 * align256(I * H / 32));
        }
    }
    std::lock_guard<std::mutex> one_load_at_a_time(mu_);
    ensure_slots(W, slot_bytes, qbytes);
    auto worker = [&](int wid) {
        const Slot& sl = slots_[(size_t)wid];
        hipStream_t st = static_cast<hipStream_t>(sl.stream);
        try {
            hipck(hipSetDevice(device_), "hipSetDevice");
            int turn = 0;
            for (int e = wid; e < n_src && !failed.load(); e += W, ++turn) {
                // two halves per slot: the host fills one while the device copies and repacks the other
                const int half = turn & 1;
                uint8_t* pinned = sl.pinned + (size_t)half * sl.bytes;
                uint8_t* dev = sl.dev + (size_t)half * sl.bytes;
                uint8_t* qdev = sl.qdev ? sl.qdev + (size_t)half * sl.qbytes : nullptr;
                hipEvent_t done = static_cast<hipEvent_t>(sl.done[half]);
                const ExpertSrc& x = experts[e];
                const size_t I = e == s.n_experts ? s.shared_inter : s.inter;
                const size_t gu_pitch = quantised && opt.pad_scale_rows ? sf_plane_pitch(H / 32) : H / 32;
                const size_t dn_pitch = quantised && opt.pad_scale_rows ? sf_plane_pitch(I / 32) : I / 32;
                // the expert before the previous one used this half: its copy has read the pinned buffer and its
                // pack kernels the device buffer
                if (turn >= 2) hipck(hipEventSynchronize(done), "hipEventSynchronize");
                size_t off = 0;
                auto stage = [&](const uint8_t* src, size_t bytes) {
                    const size_t at = off;
                    memcpy(pinned + at, src, bytes);
                    off += align256(bytes);
                    return at;
                };
                const size_t o_gw = stage(x.gate.w, x.gate.w_bytes);
                const size_t o_uw = stage(x.up.w, x.up.w_bytes);
                const size_t o_dw = stage(x.down.w, x.down.w_bytes);
                size_t o_gs = 0, o_us = 0, o_ds = 0;
                if (quantised) {
                    o_gs = off; copy_plane(pinned + off, x.gate.s, I, H / 32, gu_pitch); off += align256(I * gu_pitch);
                    o_us = off; copy_plane(pinned + off, x.up.s, I, H / 32, gu_pitch);   off += align256(I * gu_pitch);
                    o_ds = off; copy_plane(pinned + off, x.down.s, H, I / 32, dn_pitch); off += align256(H * dn_pitch);
                }
                hipck(hipMemcpyAsync(dev, pinned, off, hipMemcpyHostToDevice, st), "hipMemcpyAsync");
                ferrite_moe_expert_src src{};
                if (quantised) {
                    src.gate_w = dev + o_gw; src.gate_s = dev + o_gs;
                    src.up_w = dev + o_uw;   src.up_s = dev + o_us;
                    src.down_w = dev + o_dw; src.down_s = dev + o_ds;
                    src.gate_up_scale_pitch = (int64_t)gu_pitch;
                    src.down_scale_pitch = (int64_t)dn_pitch;
                } else {
                    const int dt = x.gate.esize == 4 ? FERRITE_DT_F32 : FERRITE_DT_BF16;
                    const size_t cb = align256(I * H / 2), sb = align256(I * H / 32);
                    uint8_t* q = qdev;
                    const size_t srcs[3] = {o_gw, o_uw, o_dw};
                    const size_t rows[3] = {I, I, H}, cols[3] = {H, H, I};
                    uint8_t* codes[3];
                    uint8_t* scales[3];
                    for (int m = 0; m < 3; ++m) {
                        codes[m] = q + (size_t)m * cb;
                        scales[m] = q + 3 * cb + (size_t)m * sb;
                        const int rc = api_->ferrite_mxfp4_quant(dev + srcs[m], dt, (int64_t)rows[m], (int64_t)cols[m],
                                                                 codes[m], scales[m], st);
                        if (rc) config_error(std::string("mxfp4_quant: rc=") + std::to_string(rc) + " " + api_->ferrite_hip_last_error());
                    }
                    src.gate_w = codes[0]; src.gate_s = scales[0];
                    src.up_w = codes[1];   src.up_s = scales[1];
                    src.down_w = codes[2]; src.down_s = scales[2];
                }
                const int rc = api_->ferrite_moe_pack_expert(&s, e, &src, packed_dev, st);
                if (rc) config_error(std::string("pack_expert: rc=") + std::to_string(rc) + " " + api_->ferrite_hip_last_error());
                hipck(hipEventRecord(done, st), "hipEventRecord");
            }
            hipck(hipStreamSynchronize(st), "hipStreamSynchronize");
        } catch (const std::exception& ex) {
            failed.store(true);
            std::lock_guard<std::mutex> g(err_mu);
            if (err.empty()) err = ex.what();
        }
        (void)hipStreamSynchronize(st);   // also after a failure: nothing of this load is left in flight
    };
    std::vector<std::thread> threads;
    for (int w = 1; w < W; ++w) threads.emplace_back(worker, w);
    try {
        load_router();
    } catch (const std::exception& ex) {
        failed.store(true);
        std::lock_guard<std::mutex> g(err_mu);
        if (err.empty()) err = ex.what();
    }
    worker(0);
    for (auto& t : threads) t.join();
    if (failed.load()) config_error(err);
    stats.seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    return stats;
}

}  // namespace ferrite
