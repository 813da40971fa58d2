// Library identity, error reporting, workspace carving, the fused MoE layer driver and the graph entry points.
// The driver only enqueues kernels on the caller's stream: no allocation, no synchronisation, no host reads
// of device data, and a launch sequence that is a function of (shape, n, mode) alone.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "internal.hpp"

#ifndef FERRITE_BUILD_ID
#define FERRITE_BUILD_ID "unstamped"
#endif

namespace fe {

static thread_local char g_last_error[256] = "";

int hip_fail(hipError_t e, const char* what) {
    snprintf(g_last_error, sizeof(g_last_error), "HIP %s: %s", what, hipGetErrorString(e));
    return FERRITE_ERR_RUNTIME;
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e, what);
    return FERRITE_OK;
}

// ---- workspace: fixed offsets for (shape, n, mode) ----
struct Workspace {
    size_t logits, probs, ids_f32, ids, counts, starts, perm_map, gather_src, active, n_active;
    size_t unit_expert, unit_row0, unit_rows, unit_first, unit_count, n_units, perm_scratch, perm_scratch_bytes, counters;
    size_t xq, xs, xq2, xs2, act, act_s, act2, act_s2, y;
    size_t total;
    int max_units, rows, unit_cap;
};

// Process-wide overrides (ferrite_hip_set_override): test hooks that replace what used to be environment reads.
static std::atomic<int> g_override_unit_rows{0};   // 0 = automatic, else 16 or 128
static std::atomic<int> g_override_y_f32{0};       // 1 = expert outputs stay f32 on the 128-row path
static std::atomic<int> g_override_head{0};        // 1 = routing as separate launches whatever the batch size

// Rows per unit: 16 (the weight-streaming kernels) while the average expert sees fewer than 16 rows; beyond that
// (256 tokens at 128 experts and top-8: measured 378 against 387 us there, 449 against 488 us at 320 tokens, 512
// against 717 us at 767) the tiled kernels, whose units hold 128 rows of one-term or 64 rows of two-term
// activations.  The override forces one family or the other (16, or 128 = the tiled kernels).
int unit_rows_for(int n, int topk, int n_experts, bool two_term) {
    const int tiled = two_term ? 64 : 128;
    const int forced = g_override_unit_rows.load(std::memory_order_relaxed);
    if (forced == 16) return 16;
    if (forced == 128) return tiled;
    return (long)n * topk >= 16L * n_experts ? tiled : 16;
}

int y_dtype_for(int unit_rows) {
    if (unit_rows < 64) return FERRITE_DT_F32;
    return g_override_y_f32.load(std::memory_order_relaxed) ? FERRITE_DT_F32 : FERRITE_DT_BF16;
}

int current_device(int* dev) {
    hipError_t e = hipGetDevice(dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    if (*dev < 0 || *dev >= kMaxDevices) return FERRITE_ERR_INVALID_ARG;
    return FERRITE_OK;
}

int raise_lds_limit(const void* kernel, size_t bytes, std::atomic<size_t>* raised) {
    static std::mutex mu;   // attribute and record change together
    std::lock_guard<std::mutex> lock(mu);
    if (bytes <= raised->load(std::memory_order_relaxed)) return FERRITE_OK;
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute");
    raised->store(bytes, std::memory_order_release);
    return FERRITE_OK;
}

static bool is_mfma_mode(int mode) { return mode == FERRITE_MODE_MFMA_FP8 || mode == FERRITE_MODE_MFMA_FP8_X2; }

static size_t bump(size_t& off, size_t bytes) {
    size_t at = off;
    off = (off + bytes + 255) / 256 * 256;
    return at;
}

static Workspace carve(const ferrite_moe_shape& s, int n, int mode) {
    Workspace w{};
    const size_t nk = (size_t)n * s.topk, E = s.n_experts, H = s.hidden;
    const int has_shared = s.shared_inter > 0;
    const size_t act_ld = s.inter > s.shared_inter ? s.inter : s.shared_inter;
    w.rows = (int)(nk + (has_shared ? n : 0));
    w.unit_cap = is_mfma_mode(mode) ? unit_rows_for(n, s.topk, s.n_experts, mode == FERRITE_MODE_MFMA_FP8_X2) : 16;
    w.max_units = max_units_for(n, s.topk, s.n_experts, has_shared, w.unit_cap);
    size_t off = 0;
    w.counters = bump(off, ((size_t)n + 1) * 4);   // first: ferrite_moe_layer_workspace_init clears it
    w.logits = bump(off, (size_t)n * E * 4);
    w.probs = bump(off, nk * 4);
    w.ids_f32 = bump(off, nk * 4);
    w.ids = bump(off, nk * 4);
    w.counts = bump(off, E * 4);
    w.starts = bump(off, (E + 1) * 4);
    w.perm_map = bump(off, nk * 4);
    w.gather_src = bump(off, nk * 4);
    w.active = bump(off, E * 4);
    w.n_active = bump(off, 4);
    w.unit_expert = bump(off, (size_t)w.max_units * 4);
    w.unit_row0 = bump(off, (size_t)w.max_units * 4);
    w.unit_rows = bump(off, (size_t)w.max_units * 4);
    w.unit_first = bump(off, (size_t)w.max_units * 4);
    w.unit_count = bump(off, (size_t)w.max_units * 4);
    w.n_units = bump(off, 4);
    w.perm_scratch_bytes = perm_scratch_bytes(n, s.n_experts);
    w.perm_scratch = bump(off, w.perm_scratch_bytes);
    if (is_mfma_mode(mode)) {
        const size_t xs_row = ((H / 128 + 3) / 4) * 16, as_row = ((act_ld / 128 + 3) / 4) * 16;
        w.xq = bump(off, (size_t)n * H);
        w.xs = bump(off, (size_t)n * xs_row);
        w.act = bump(off, (size_t)w.rows * act_ld);
        w.act_s = bump(off, (size_t)w.rows * as_row);
        if (mode == FERRITE_MODE_MFMA_FP8_X2) {
            w.xq2 = bump(off, (size_t)n * H);
            w.xs2 = bump(off, (size_t)n * xs_row);
            w.act2 = bump(off, (size_t)w.rows * act_ld);
            w.act_s2 = bump(off, (size_t)w.rows * as_row);
        }
    } else {
        w.act = bump(off, (size_t)w.rows * act_ld * 4);
    }
    w.y = bump(off, (size_t)w.rows * H * 4);
    w.total = off;
    return w;
}

static int check_shape(const ferrite_moe_shape* s, int n, int mode) {
    if (!s || n <= 0) return FERRITE_ERR_INVALID_ARG;
    if (s->hidden <= 0 || s->n_experts <= 0 || s->topk <= 0 || s->topk > s->n_experts || s->inter <= 0 ||
        s->shared_inter < 0)
        return FERRITE_ERR_INVALID_ARG;
    if (mode != FERRITE_MODE_F32_CHECK && !is_mfma_mode(mode)) return FERRITE_ERR_INVALID_ARG;
    if (s->hidden % 32 || s->inter % 32 || s->shared_inter % 32) return FERRITE_ERR_INVALID_ARG;
    if (is_mfma_mode(mode) && (s->hidden % 128 || s->inter % 128 || s->shared_inter % 128)) return FERRITE_DECLINED;
    if (n > 65535) return FERRITE_DECLINED;   // token index on grid.y of several kernels: split the batch
    // the routing kernels' own limits, for the fused head and the separate launches alike
    return check_routing_params(s->n_experts, s->topk, s->n_group, s->topk_group);
}

}  // namespace fe

using namespace fe;

extern "C" const char* ferrite_kernel_build_id(void) { return FERRITE_BUILD_ID; }
extern "C" unsigned ferrite_kernel_abi_version(void) { return FERRITE_ABI_VERSION; }
extern "C" const char* ferrite_hip_last_error(void) { return g_last_error; }

extern "C" int ferrite_hip_set_override(int which, int value) {
    if (which == FERRITE_OVERRIDE_UNIT_ROWS) {
        if (value != 0 && value != 16 && value != 128) return FERRITE_ERR_INVALID_ARG;
        g_override_unit_rows.store(value);
        return FERRITE_OK;
    }
    if (which == FERRITE_OVERRIDE_HEAD) {
        if (value != 0 && value != 1) return FERRITE_ERR_INVALID_ARG;
        g_override_head.store(value);
        return FERRITE_OK;
    }
    if (which == FERRITE_OVERRIDE_PREFILL_TILE) {
        if (value < 0 || value > 3) return FERRITE_ERR_INVALID_ARG;
        set_prefill_variant(value);
        return FERRITE_OK;
    }
    if (which == FERRITE_OVERRIDE_Y_F32) {
        if (value != 0 && value != 1) return FERRITE_ERR_INVALID_ARG;
        g_override_y_f32.store(value);
        return FERRITE_OK;
    }
    return FERRITE_ERR_INVALID_ARG;
}

static int static_workspace(void** out);

extern "C" int ferrite_hip_warmup(void) {
    int rc;
    if ((rc = warmup_route())) return rc;
    if ((rc = warmup_experts_mfma())) return rc;
    void* ws = nullptr;
    return static_workspace(&ws);   // resolves this device's copy of the built-in workspace
}

extern "C" int ferrite_moe_layer_check(const ferrite_moe_shape* shape, int n, int mode) { return check_shape(shape, n, mode); }

extern "C" int ferrite_moe_layer_unit_rows(const ferrite_moe_shape* shape, int n, int mode) {
    if (check_shape(shape, n, mode)) return 0;
    return carve(*shape, n, mode).unit_cap;
}

extern "C" size_t ferrite_moe_layer_workspace_bytes(const ferrite_moe_shape* shape, int n, int mode) {
    if (check_shape(shape, n, mode)) return 0;
    return carve(*shape, n, mode).total;
}

extern "C" int ferrite_moe_layer_workspace_init(const ferrite_moe_shape* shape, int n, int mode, void* workspace,
                                                size_t workspace_bytes, ferrite_stream_t stream) {
    int rc = check_shape(shape, n, mode);
    if (rc) return rc;
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255)) return FERRITE_ERR_INVALID_ARG;
    Workspace w = carve(*shape, n, mode);
    if (workspace_bytes < w.total) return FERRITE_ERR_WORKSPACE;
    return launch_zero_i32(reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + w.counters), n + 1,
                           as_stream(stream));
}

extern "C" int ferrite_moe_layer_workspace_view(const ferrite_moe_shape* shape, int n, int mode, void* workspace,
                                                ferrite_moe_workspace_view* v) {
    int rc = check_shape(shape, n, mode);
    if (rc) return rc;
    if (!workspace || !v) return FERRITE_ERR_INVALID_ARG;
    Workspace w = carve(*shape, n, mode);
    char* b = static_cast<char*>(workspace);
    v->logits = reinterpret_cast<float*>(b + w.logits);
    v->probs = reinterpret_cast<float*>(b + w.probs);
    v->ids_f32 = reinterpret_cast<float*>(b + w.ids_f32);
    v->ids = reinterpret_cast<int32_t*>(b + w.ids);
    v->counts = reinterpret_cast<int32_t*>(b + w.counts);
    v->starts = reinterpret_cast<int32_t*>(b + w.starts);
    v->perm_map = reinterpret_cast<int32_t*>(b + w.perm_map);
    v->gather_src = reinterpret_cast<int32_t*>(b + w.gather_src);
    v->active = reinterpret_cast<int32_t*>(b + w.active);
    v->n_active = reinterpret_cast<int32_t*>(b + w.n_active);
    v->y = reinterpret_cast<float*>(b + w.y);
    return FERRITE_OK;
}

static int mark(void* const* ev, int i, hipStream_t st) {
    if (!ev || !ev[i]) return FERRITE_OK;
    hipError_t e = hipEventRecord(static_cast<hipEvent_t>(ev[i]), st);
    return e == hipSuccess ? FERRITE_OK : hip_fail(e, "hipEventRecord");
}

// norm_w (may be NULL): x is the un-normalised f32 stream and the fused head applies rmsnorm(x, norm_w, norm_eps) to
// it on the fly; only legal where head_norm_supported() says so.  hc (may be NULL): the combine applies hc_post to
// the layer's output on the way out; out is then [n, nh, H] f32.
static int moe_layer_impl(const ferrite_moe_shape* shape, const ferrite_moe_weights* wts, const uint8_t* packed,
                          const void* x, int x_dtype, int n, void* out, int out_dtype, int mode, void* workspace,
                          size_t workspace_bytes, ferrite_stream_t stream, void* const* ev,
                          const float* norm_w = nullptr, float norm_eps = 0.0f, const HcPostArgs* hc = nullptr,
                          bool clear_counters = false) {
    int rc = check_shape(shape, n, mode);
    if (rc) return rc;
    // the packed buffer carries the router weight (transposed); the checkpoint-layout one is read only without it
    if (!wts || (!packed && !wts->router_w) || !x || !out || !workspace) return FERRITE_ERR_INVALID_ARG;
    if ((reinterpret_cast<uintptr_t>(workspace) & 255) || (reinterpret_cast<uintptr_t>(x) & 15) ||
        (reinterpret_cast<uintptr_t>(out) & 15))
        return FERRITE_ERR_INVALID_ARG;
    if (x_dtype != FERRITE_DT_F32 && x_dtype != FERRITE_DT_BF16) return FERRITE_ERR_INVALID_ARG;
    if (out_dtype != FERRITE_DT_F32 && out_dtype != FERRITE_DT_BF16) return FERRITE_ERR_INVALID_ARG;
    const ferrite_moe_shape& s = *shape;
    if (mode == FERRITE_MODE_F32_CHECK) {
        if (x_dtype != FERRITE_DT_F32) return FERRITE_ERR_INVALID_ARG;
        if (!wts->gate_w || !wts->gate_s || !wts->up_w || !wts->up_s || !wts->down_w || !wts->down_s)
            return FERRITE_ERR_INVALID_ARG;
        if (s.shared_inter > 0 && (!wts->sh_gate_w || !wts->sh_gate_s || !wts->sh_up_w || !wts->sh_up_s ||
                                   !wts->sh_down_w || !wts->sh_down_s))
            return FERRITE_ERR_INVALID_ARG;
    } else if (!packed) {
        return FERRITE_ERR_INVALID_ARG;
    }
    Workspace w = carve(s, n, mode);
    if (workspace_bytes < w.total) return FERRITE_ERR_WORKSPACE;
    char* b = static_cast<char*>(workspace);
    hipStream_t st = as_stream(stream);
    const int has_shared = s.shared_inter > 0;
    if (norm_w && !(packed != nullptr && head_supported(n, s.hidden, s.n_experts) && is_mfma_mode(mode) &&
                    x_dtype == FERRITE_DT_F32 && head_norm_supported(n, s.hidden, s.n_experts)))
        return FERRITE_ERR_INVALID_ARG;
    // every argument has been checked: from here on the call only enqueues
    if (clear_counters &&
        (rc = launch_zero_i32(reinterpret_cast<int32_t*>(b + w.counters), n + 1, st)))
        return rc;

    float* logits = reinterpret_cast<float*>(b + w.logits);
    float* probs = reinterpret_cast<float*>(b + w.probs);
    float* ids_f32 = reinterpret_cast<float*>(b + w.ids_f32);
    int32_t* ids = reinterpret_cast<int32_t*>(b + w.ids);
    int32_t* perm_map = reinterpret_cast<int32_t*>(b + w.perm_map);
    int32_t* gather_src = reinterpret_cast<int32_t*>(b + w.gather_src);
    void* y = b + w.y;
    const int y_dtype = is_mfma_mode(mode) ? y_dtype_for(w.unit_cap) : FERRITE_DT_F32;
    const bool x2 = mode == FERRITE_MODE_MFMA_FP8_X2;
    auto at = [&](size_t off) { return reinterpret_cast<uint8_t*>(b + off); };
    const ActPlanes xq = is_mfma_mode(mode) ? ActPlanes{at(w.xq), at(w.xs), x2 ? at(w.xq2) : nullptr, x2 ? at(w.xs2) : nullptr}
                                            : ActPlanes{nullptr, nullptr, nullptr, nullptr};

    UnitTables units{reinterpret_cast<int32_t*>(b + w.unit_expert), reinterpret_cast<int32_t*>(b + w.unit_row0),
                     reinterpret_cast<int32_t*>(b + w.unit_rows), reinterpret_cast<int32_t*>(b + w.unit_first),
                     reinterpret_cast<int32_t*>(b + w.unit_count), reinterpret_cast<int32_t*>(b + w.n_units), w.unit_cap,
                     w.max_units};
    if ((rc = mark(ev, 0, st))) return rc;
    const bool fused_head = packed != nullptr && head_supported(n, s.hidden, s.n_experts) &&
                            !(g_override_head.load(std::memory_order_relaxed) == 1 && !norm_w);
    if (norm_w && !(fused_head && is_mfma_mode(mode) && x_dtype == FERRITE_DT_F32 &&
                    head_norm_supported(n, s.hidden, s.n_experts)))
        return FERRITE_ERR_INVALID_ARG;
    if (fused_head) {
        // 1-3 (+ activation quantisation) as one launch
        PackedLayout L = packed_layout(s);
        const int fuse_perm = 1;   // the block that routes the last token builds the tables
        if ((rc = launch_moe_head(x, x_dtype, reinterpret_cast<const float*>(packed + L.router_t), wts->router_bias, s,
                                  n, logits, probs, ids_f32, ids, xq, reinterpret_cast<int32_t*>(b + w.counters),
                                  reinterpret_cast<int32_t*>(b + w.counts), reinterpret_cast<int32_t*>(b + w.starts),
                                  perm_map, gather_src, reinterpret_cast<int32_t*>(b + w.active),
                                  reinterpret_cast<int32_t*>(b + w.n_active), &units, fuse_perm, norm_w, norm_eps, st)))
            return rc;
        if ((rc = mark(ev, 1, st))) return rc;
        if ((rc = mark(ev, 2, st))) return rc;
        if (!fuse_perm &&
            (rc = launch_permute(ids, n, s.topk, s.n_experts, reinterpret_cast<int32_t*>(b + w.counts),
                                 reinterpret_cast<int32_t*>(b + w.starts), perm_map, gather_src,
                                 reinterpret_cast<int32_t*>(b + w.active), reinterpret_cast<int32_t*>(b + w.n_active),
                                 b + w.perm_scratch, w.perm_scratch_bytes, &units, has_shared, st)))
            return rc;
        if ((rc = mark(ev, 3, st))) return rc;
        if ((rc = mark(ev, 4, st))) return rc;
    } else {
    // 1. router logits: the reference's sequential-k f32 chain (exec/lib.rs:1107)
    if (packed != nullptr && s.hidden % 128 == 0) {
        PackedLayout L = packed_layout(s);
        rc = launch_router_chain(x, x_dtype, reinterpret_cast<const float*>(packed + L.router_t), n, s.hidden,
                                 s.n_experts, logits, st);
        if (rc == FERRITE_DECLINED) {
            if (!wts->router_w) return FERRITE_ERR_INVALID_ARG;   // this shape needs the checkpoint-layout router
            rc = launch_matmul_exact(x, x_dtype, wts->router_w, nullptr, logits, n, s.hidden, s.n_experts, st);
        }
    } else {
        rc = launch_matmul_exact(x, x_dtype, wts->router_w, nullptr, logits, n, s.hidden, s.n_experts, st);
    }
    if (rc) return rc;
    if ((rc = mark(ev, 1, st))) return rc;
    // 2. routing (exec/lib.rs:1109-1116); a NULL bias is the reference's zero bias
    if ((rc = ferrite_moe_route(logits, wts->router_bias, n, s.n_experts, s.topk, s.n_group, s.topk_group,
                                s.routed_scaling, probs, ids_f32, ids, stream)))
        return rc;
    if ((rc = mark(ev, 2, st))) return rc;
    // 3. permutation by expert + unit tables
    if ((rc = launch_permute(ids, n, s.topk, s.n_experts, reinterpret_cast<int32_t*>(b + w.counts),
                             reinterpret_cast<int32_t*>(b + w.starts), perm_map, gather_src,
                             reinterpret_cast<int32_t*>(b + w.active), reinterpret_cast<int32_t*>(b + w.n_active),
                             b + w.perm_scratch, w.perm_scratch_bytes, &units, has_shared, st)))
        return rc;
    if ((rc = mark(ev, 3, st))) return rc;
    if (xq.q) {
        if ((rc = launch_act_quant(x, x_dtype, n, s.hidden, xq.q, xq.s, xq.q2, xq.s2, 1, st))) return rc;
    }
    if ((rc = mark(ev, 4, st))) return rc;
    }
    // 4-5. expert FFNs in grouped order, shared expert as the trailing rows
    if (mode == FERRITE_MODE_F32_CHECK) {
        float* act = reinterpret_cast<float*>(b + w.act);
        if ((rc = launch_gate_up_f32(s, *wts, static_cast<const float*>(x), n, ids, gather_src, act, st))) return rc;
        if ((rc = mark(ev, 5, st))) return rc;
        if ((rc = launch_down_f32(s, *wts, act, n, ids, gather_src, static_cast<float*>(y), st))) return rc;
    } else {
        const ActPlanes act{at(w.act), at(w.act_s), x2 ? at(w.act2) : nullptr, x2 ? at(w.act_s2) : nullptr};
        if ((rc = launch_gate_up_mfma(s, packed, xq, n, gather_src, units, act, st,
                                      ev ? static_cast<hipEvent_t>(ev[8]) : nullptr,
                                      ev ? static_cast<hipEvent_t>(ev[9]) : nullptr)))
            return rc;
        if ((rc = mark(ev, 5, st))) return rc;
        if ((rc = launch_down_mfma(s, packed, act, n, units, y, y_dtype, st))) return rc;
    }
    if ((rc = mark(ev, 6, st))) return rc;
    // 6. weighted combine in slot order + shared expert (exec/lib.rs:1154-1164)
    if ((rc = launch_combine(y, y_dtype, probs, perm_map, n, s.topk, s.hidden, has_shared, out, out_dtype, st, hc))) return rc;
    return mark(ev, 7, st);
}

extern "C" int ferrite_moe_layer_mxfp4(const ferrite_moe_shape* shape, const ferrite_moe_weights* wts,
                                       const uint8_t* packed, const void* x, int x_dtype, int n, void* out,
                                       int out_dtype, int mode, void* workspace, size_t workspace_bytes,
                                       ferrite_stream_t stream) {
    return moe_layer_impl(shape, wts, packed, x, x_dtype, n, out, out_dtype, mode, workspace, workspace_bytes, stream,
                          nullptr);
}

extern "C" int ferrite_moe_layer_mxfp4_timed(const ferrite_moe_shape* shape, const ferrite_moe_weights* wts,
                                             const uint8_t* packed, const void* x, int x_dtype, int n, void* out,
                                             int out_dtype, int mode, void* workspace, size_t workspace_bytes,
                                             ferrite_stream_t stream, void* const* stage_events) {
    return moe_layer_impl(shape, wts, packed, x, x_dtype, n, out, out_dtype, mode, workspace, workspace_bytes, stream,
                          stage_events);
}

// ---- the layer for callers that cannot allocate: its workspace is a file-scope device array ----
// Each GPU the library runs on holds its own copy of the array, at its own address, until the process ends.  The
// array's name is a host-side stand-in for it, not a device address: host code uses the address that
// hipGetSymbolAddress returns for the current device, kept per device.
static __device__ __align__(256) unsigned char scratch[FERRITE_STATIC_WORKSPACE_BYTES];

static int static_workspace(void** out) {
    static std::mutex mu;
    static std::atomic<void*> ptrs[kMaxDevices] = {};
    int dev = 0;
    if (int rc = current_device(&dev)) return rc;
    void* p = ptrs[dev].load(std::memory_order_acquire);   // the usual case: looked up before, no lock
    if (!p) {
        std::lock_guard<std::mutex> lock(mu);
        p = ptrs[dev].load(std::memory_order_relaxed);
        if (!p) {
            hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
            if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress");
            if (!p || (reinterpret_cast<uintptr_t>(p) & 255)) return FERRITE_ERR_RUNTIME;
            ptrs[dev].store(p, std::memory_order_release);
        }
    }
    *out = p;
    return FERRITE_OK;
}

extern "C" int ferrite_moe_layer_mxfp4_static(const ferrite_moe_shape* shape, const ferrite_moe_weights* wts,
                                              const uint8_t* packed, const void* x, int x_dtype, int n, void* out,
                                              int out_dtype, int mode, ferrite_stream_t stream) {
    int rc = check_shape(shape, n, mode);
    if (rc) return rc;
    const Workspace w = carve(*shape, n, mode);
    if (w.total > FERRITE_STATIC_WORKSPACE_BYTES) {
        snprintf(g_last_error, sizeof(g_last_error),
                 "ferrite_moe_layer_mxfp4_static: this call needs %zu bytes of workspace, the built-in one holds %zu",
                 w.total, (size_t)FERRITE_STATIC_WORKSPACE_BYTES);
        return FERRITE_ERR_WORKSPACE;
    }
    void* ws = nullptr;
    if ((rc = static_workspace(&ws))) return rc;
    // The array keeps what the last call left in it.  Only the arrival counters have to start at zero; a call that
    // ran to its end leaves them so, one that was cut short may not have: cleared by a kernel (capturable) at the
    // head of the call's launches, once its arguments have passed every check.
    return moe_layer_impl(shape, wts, packed, x, x_dtype, n, out, out_dtype, mode, ws, FERRITE_STATIC_WORKSPACE_BYTES,
                          stream, nullptr, nullptr, 0.0f, nullptr, /*clear_counters=*/true);
}

// ---- rmsnorm -> layer -> hc_post (exec/lib.rs:487-492) ----
static size_t block_extra(const ferrite_moe_shape& s, int n) { return ((size_t)n * s.hidden * 4 + 255) / 256 * 256; }

extern "C" size_t ferrite_moe_block_workspace_bytes(const ferrite_moe_shape* shape, int n, int mode) {
    if (check_shape(shape, n, mode)) return 0;
    return carve(*shape, n, mode).total + 2 * block_extra(*shape, n);
}

extern "C" int ferrite_moe_block_mxfp4(const ferrite_moe_shape* shape, const ferrite_moe_weights* wts,
                                       const uint8_t* packed, const float* li, const ferrite_moe_block_args* blk, int n,
                                       float* out, int mode, void* workspace, size_t workspace_bytes,
                                       ferrite_stream_t stream) {
    int rc = check_shape(shape, n, mode);
    if (rc) return rc;
    if (!li || !blk || !out || !workspace || !blk->norm_w) return FERRITE_ERR_INVALID_ARG;
    const bool with_hc_post = blk->residual != nullptr;
    if (with_hc_post && (!blk->post || !blk->comb || blk->nh <= 0)) return FERRITE_ERR_INVALID_ARG;
    const ferrite_moe_shape& s = *shape;
    const size_t layer_bytes = carve(s, n, mode).total, extra = block_extra(s, n);
    if (workspace_bytes < layer_bytes + 2 * extra) return FERRITE_ERR_WORKSPACE;
    char* b = static_cast<char*>(workspace);
    float* hfn = reinterpret_cast<float*>(b + layer_bytes);
    // The two neighbours fold into the layer's own launches where nothing else needs their results in memory:
    // rmsnorm into the fused routing head (MFMA modes: the expert GEMMs take the quantised activations that the head
    // writes), hc_post into the combine (a per-element function of the layer's output).
    // (the head reads norm_w with 16-byte loads; a misaligned one takes the separate rmsnorm launch, which checks)
    const bool fused_norm = is_mfma_mode(mode) && packed != nullptr && head_norm_supported(n, s.hidden, s.n_experts) &&
                            (reinterpret_cast<uintptr_t>(blk->norm_w) & 15) == 0 &&
                            g_override_head.load(std::memory_order_relaxed) != 1;
    // (hc_post only for decode-sized batches, where it saves a launch: at 4096 tokens the combine with the 4-stream
    // epilogue took 221 us against 57 + 104 us for the two kernels)
    const bool fused_hc = with_hc_post && n <= 256 && blk->nh <= 8 && (reinterpret_cast<uintptr_t>(blk->residual) & 15) == 0;
    const HcPostArgs hc{blk->residual, blk->post, blk->comb, blk->nh};
    float* ffn_out = (with_hc_post && !fused_hc) ? reinterpret_cast<float*>(b + layer_bytes + extra) : out;
    const float* xin = li;
    if (!fused_norm) {
        if ((rc = ferrite_rmsnorm_f32(li, blk->norm_w, blk->eps, hfn, n, s.hidden, stream))) return rc;
        xin = hfn;
    }
    if ((rc = moe_layer_impl(shape, wts, packed, xin, FERRITE_DT_F32, n, ffn_out, FERRITE_DT_F32, mode, workspace,
                             layer_bytes, stream, nullptr, fused_norm ? blk->norm_w : nullptr, blk->eps,
                             fused_hc ? &hc : nullptr)))
        return rc;
    if (!with_hc_post || fused_hc) return FERRITE_OK;
    return ferrite_hc_post_f32(ffn_out, blk->residual, blk->post, blk->comb, out, n, blk->nh, s.hidden, stream);
}

// ---- graph capture (ferrite_graph_begin/end/instantiate/launch, cuda.rs:284-287) ----
extern "C" int ferrite_graph_begin(ferrite_stream_t stream) {
    hipError_t e = hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal);
    return e == hipSuccess ? FERRITE_OK : hip_fail(e, "hipStreamBeginCapture");
}

extern "C" int ferrite_graph_end(ferrite_stream_t stream, void** graph_exec_out) {
    if (!graph_exec_out) return FERRITE_ERR_INVALID_ARG;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(as_stream(stream), &graph);
    if (e != hipSuccess) return hip_fail(e, "hipStreamEndCapture");
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return hip_fail(e, "hipGraphInstantiate");
    *graph_exec_out = exec;
    return FERRITE_OK;
}

extern "C" int ferrite_graph_launch(void* graph_exec, ferrite_stream_t stream) {
    if (!graph_exec) return FERRITE_ERR_INVALID_ARG;
    hipError_t e = hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), as_stream(stream));
    return e == hipSuccess ? FERRITE_OK : hip_fail(e, "hipGraphLaunch");
}

extern "C" int ferrite_graph_destroy(void* graph_exec) {
    if (!graph_exec) return FERRITE_OK;
    hipError_t e = hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec));
    return e == hipSuccess ? FERRITE_OK : hip_fail(e, "hipGraphExecDestroy");
}
