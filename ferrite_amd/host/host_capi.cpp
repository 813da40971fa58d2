#include "ferrite_host.h"

#include <cstdio>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "checkpoint.hpp"

using namespace ferrite;

struct ferrite_ckpt_shard {
    SafetensorsIndex index;
    std::unique_ptr<MappedFile> file;
};

struct ferrite_ckpt {
    std::vector<std::unique_ptr<ferrite_ckpt_shard>> shards;   // at least one; a tensor is taken from the first that names it
    const TensorView* find(const std::string& name) const {
        for (const auto& sh : shards)
            if (const TensorView* v = sh->index.find(name)) return v;
        return nullptr;
    }
    // the loader (library handle, staging buffers, streams) is kept between layers of the same shard
    std::unique_ptr<MoeCheckpointLoader> loader;
    std::string loader_so;
    int loader_device = -1;
};

static void set_err(char* err, size_t errlen, const char* msg) {
    if (err && errlen) snprintf(err, errlen, "%s", msg);
}

extern "C" ferrite_ckpt* ferrite_ckpt_open(const char* path, char* err, size_t errlen) {
    try {
        if (!path) throw FerriteError(FerriteError::InvalidArg, "path is null");
        std::unique_ptr<ferrite_ckpt> ck(new ferrite_ckpt);
        std::unique_ptr<ferrite_ckpt_shard> sh(new ferrite_ckpt_shard);
        sh->index = SafetensorsIndex::read_header(path);
        sh->file.reset(new MappedFile(path));
        ck->shards.push_back(std::move(sh));
        return ck.release();
    } catch (const std::exception& e) {
        set_err(err, errlen, e.what());
        return nullptr;
    }
}

extern "C" int ferrite_ckpt_add_shard(ferrite_ckpt* ck, const char* path, char* err, size_t errlen) {
    try {
        if (!ck || !path) throw FerriteError(FerriteError::InvalidArg, "null argument");
        std::unique_ptr<ferrite_ckpt_shard> sh(new ferrite_ckpt_shard);
        sh->index = SafetensorsIndex::read_header(path);
        sh->file.reset(new MappedFile(path));
        ck->shards.push_back(std::move(sh));
        return 0;
    } catch (const std::exception& e) {
        set_err(err, errlen, e.what());
        return 1;
    }
}

extern "C" void ferrite_ckpt_close(ferrite_ckpt* ck) { delete ck; }

extern "C" int64_t ferrite_ckpt_num_tensors(const ferrite_ckpt* ck) {
    if (!ck) return -1;
    int64_t n = 0;
    for (const auto& sh : ck->shards) n += (int64_t)sh->index.tensors.size();
    return n;
}

extern "C" uint64_t ferrite_ckpt_data_start(const ferrite_ckpt* ck) { return ck ? ck->shards[0]->index.data_start : 0; }

extern "C" int ferrite_ckpt_tensor(const ferrite_ckpt* ck, const char* name, char dtype[16], int64_t shape[8], int* ndim,
                                   uint64_t* begin, uint64_t* end) {
    if (!ck || !name) return 2;
    const TensorView* v = ck->find(name);
    if (!v) return 1;
    if (dtype) snprintf(dtype, 16, "%s", v->dtype.c_str());
    if (ndim) *ndim = (int)v->shape.size();
    if (shape)
        for (size_t i = 0; i < v->shape.size() && i < 8; ++i) shape[i] = (int64_t)v->shape[i];
    if (begin) *begin = v->begin;
    if (end) *end = v->end;
    return 0;
}

extern "C" int ferrite_ckpt_validate_moe(const ferrite_ckpt* ck, int naming, const char* prefix,
                                         const ferrite_moe_shape* shape, char* report, size_t report_len) {
    if (!ck || !prefix || !shape || naming < 0 || naming > 1) return -1;
    // a spec is satisfied by the first shard that names its tensor
    std::vector<std::string> missing;
    for (const TensorSpec& spec : moe_layer_specs(static_cast<MoeNaming>(naming), prefix, *shape)) {
        bool found = false;
        for (const auto& sh : ck->shards) {
            if (!sh->index.find(spec.name)) continue;
            found = true;
            for (const auto& m : sh->index.validate({spec})) missing.push_back(m);
            break;
        }
        if (!found) missing.push_back(spec.name);
    }
    if (report && report_len) {
        std::string all;
        for (const auto& m : missing) all += m + "\n";
        snprintf(report, report_len, "%s", all.c_str());
    }
    return (int)missing.size();
}

extern "C" int ferrite_ckpt_load_moe_layer(const ferrite_ckpt* ck, const char* hip_so_path, int device, int naming,
                                           const char* prefix, const ferrite_moe_shape* shape, void* packed_dev,
                                           void* router_bias_dev, int workers, int pad_scale_rows, double stats[4],
                                           char* err, size_t errlen) {
    try {
        if (!ck || !hip_so_path || !prefix || !shape || naming < 0 || naming > 1)
            throw FerriteError(FerriteError::InvalidArg, "null or out-of-range argument");
        ferrite_ckpt* mck = const_cast<ferrite_ckpt*>(ck);
        if (!mck->loader || mck->loader_so != hip_so_path || mck->loader_device != device) {
            mck->loader.reset(new MoeCheckpointLoader(hip_so_path, device));
            mck->loader_so = hip_so_path;
            mck->loader_device = device;
        }
        const MoeCheckpointLoader& loader = *mck->loader;
        LoadOptions opt;
        if (workers > 0) opt.workers = workers;
        opt.pad_scale_rows = pad_scale_rows != 0;
        std::vector<CheckpointShard> shards;
        for (const auto& sh : ck->shards) shards.push_back(CheckpointShard{sh->file.get(), &sh->index});
        const LoadStats st = loader.load_layer(shards, static_cast<MoeNaming>(naming), prefix, *shape,
                                               static_cast<uint8_t*>(packed_dev), static_cast<float*>(router_bias_dev), opt);
        if (stats) {
            stats[0] = (double)st.source_bytes;
            stats[1] = (double)st.packed_bytes;
            stats[2] = st.seconds;
            stats[3] = (double)st.workers;
        }
        return 0;
    } catch (const std::exception& e) {
        set_err(err, errlen, e.what());
        return 1;
    }
}
