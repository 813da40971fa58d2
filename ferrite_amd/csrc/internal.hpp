// Declarations shared between the translation units of libferrite_hip.so (not part of the public ABI).
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
#include <stddef.h>
#include <stdint.h>

#include "../../include/ferrite_hip.h"

namespace fe {

// Records a failed HIP runtime call for ferrite_hip_last_error() and returns FERRITE_ERR_RUNTIME.
int hip_fail(hipError_t e, const char* what);
// Checks the launch that was just issued on this thread.
int check_launch(const char* what);

inline hipStream_t as_stream(ferrite_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// A unit is up to `unit_rows` consecutive rows of the grouped order that share one expert; the expert GEMM
// kernels are launched over a fixed upper bound of units and read the live count from n_units.
struct UnitTables {
    int32_t* unit_expert;  // [max_units] expert id (n_experts = the shared expert)
    int32_t* unit_row0;    // [max_units] first grouped row
    int32_t* unit_rows;    // [max_units] rows in the unit (1..unit_rows)
    int32_t* unit_first;   // [max_units] index of the first unit of this unit's expert (may be NULL: not written)
    int32_t* unit_count;   // [max_units] number of units of this unit's expert
    int32_t* n_units;      // [1]
    int unit_rows_cap;     // rows per unit (column tile of the GEMM)
    int max_units;
};

inline int max_units_for(int n, int topk, int n_experts, int has_shared, int unit_rows) {
    long assign = (long)n * topk;
    long active_max = assign < n_experts ? assign : n_experts;
    long u = assign / unit_rows + active_max + (has_shared ? (n + unit_rows - 1) / unit_rows : 0);
    return (int)u;
}

// Rows per unit for a layer call: the tiled kernels (units of 128 rows, 64 with two-term activations) once the
// average expert sees enough rows to fill them, 16-row units (weights streamed once per unit) below that.  A
// process-wide override (ferrite_hip_set_override, a test hook) forces either; nothing here reads the environment.
int unit_rows_for(int n, int topk, int n_experts, bool two_term);
// Element type of the expert outputs `y` in the workspace: bf16 for the tiled kernels (prefill-sized batches, where the
// y round trip through HBM is a tenth of the layer), f32 otherwise.  The FERRITE_OVERRIDE_Y_F32 override forces f32.
int y_dtype_for(int unit_rows);

// Kernels that need more than 64 KiB of dynamic LDS must have the limit raised once per device (a function
// attribute, not a stream operation, and therefore not something to do inside a stream capture:
// ferrite_hip_warmup() raises every kernel's limit to the most it can ever ask for).  LdsLimit<kernel>::ensure()
// is the per-launch check: an atomic read on the fast path, a mutex around the attribute call otherwise.
constexpr size_t kLdsCap = 160 * 1024;
constexpr int kMaxDevices = 16;
int current_device(int* dev);
int raise_lds_limit(const void* kernel, size_t bytes, std::atomic<size_t>* raised);

template <auto Kernel>
struct LdsLimit {
    static inline std::atomic<size_t> raised[kMaxDevices] = {};
    static int ensure(size_t bytes) {
        if (bytes <= 64 * 1024) return FERRITE_OK;
        if (bytes > kLdsCap) return FERRITE_DECLINED;
        int dev = 0;
        if (int rc = current_device(&dev)) return rc;
        if (bytes <= raised[dev].load(std::memory_order_acquire)) return FERRITE_OK;
        return raise_lds_limit(reinterpret_cast<const void*>(Kernel), bytes, &raised[dev]);
    }
};

// Per translation unit: raise the LDS limit of every kernel in it that may exceed 64 KiB (ferrite_hip_warmup).
int warmup_route();
int warmup_experts_mfma();

// Activation buffers of the expert GEMMs: e4m3 codes and operand-order scales, one plane, or two for two-term
// activations (q2 / s2 null otherwise).
struct ActPlanes {
    uint8_t *q, *s, *q2, *s2;
};

// route.hip
int launch_matmul_exact(const void* x, int x_dtype, const float* w, const float* bias, float* out, int n, int k,
                        int o, hipStream_t st);
int launch_permute(const int32_t* ids, int n, int topk, int n_experts, int32_t* counts, int32_t* starts,
                   int32_t* perm_map, int32_t* gather_src, int32_t* active, int32_t* n_active, void* scratch,
                   size_t scratch_bytes, const UnitTables* units, int has_shared, hipStream_t st);

int check_routing_params(int e, int topk, int n_group, int topk_group);
size_t perm_scratch_bytes(int n_tokens, int n_experts);   // masks + offsets of the three-phase permutation
bool head_supported(int n, int H, int E);
bool head_norm_supported(int n, int H, int E);   // ... with rmsnorm of the (f32) input fused in front
int launch_moe_head(const void* x, int x_dtype, const float* router_t, const float* bias, const ferrite_moe_shape& s,
                    int n, float* logits, float* probs, float* ids_f32, int32_t* ids, const ActPlanes& xq,
                    int32_t* counters, int32_t* counts, int32_t* starts, int32_t* perm_map, int32_t* gather_src,
                    int32_t* active, int32_t* n_active, const UnitTables* units, int fuse_perm, const float* norm_w,
                    float eps, hipStream_t st);
int launch_router_chain(const void* x, int x_dtype, const float* router_t, int n, int H, int E, float* logits,
                        hipStream_t st);
int launch_router_transpose(const float* w, int E, int H, float* dst, hipStream_t st);
int launch_zero_i32(int32_t* p, int count, hipStream_t st);

// experts_f32.hip (check mode)
int launch_gate_up_f32(const ferrite_moe_shape& s, const ferrite_moe_weights& w, const float* x, int n,
                       const int32_t* ids, const int32_t* gather_src, float* act, hipStream_t st);
int launch_down_f32(const ferrite_moe_shape& s, const ferrite_moe_weights& w, const float* act, int n,
                    const int32_t* ids, const int32_t* gather_src, float* y, hipStream_t st);
// The hyper-connection update behind the layer, for a combine that applies it on the way out (f32 output only):
// residual [n, nh, H], post [n, nh], comb [n, nh, nh]; out is then [n, nh, H].
struct HcPostArgs {
    const float *residual, *post, *comb;
    int nh;
};
int launch_combine(const void* y, int y_dtype, const float* probs, const int32_t* perm_map, int n, int topk,
                   int hidden, int has_shared, void* out, int out_dtype, hipStream_t st,
                   const HcPostArgs* hc = nullptr);

// experts_mfma.hip
struct PackedLayout {
    // byte offsets into the packed buffer
    size_t gu_codes, gu_scales, dn_codes, dn_scales;           // routed experts
    size_t sh_gu_codes, sh_gu_scales, sh_dn_codes, sh_dn_scales; // shared expert
    size_t gu_codes_per_expert, gu_scales_per_expert, dn_codes_per_expert, dn_scales_per_expert;
    size_t router_t;                                           // k-blocked transpose of the router weight
    size_t total;
};
PackedLayout packed_layout(const ferrite_moe_shape& s);
int launch_gate_up_mfma(const ferrite_moe_shape& s, const uint8_t* packed, const ActPlanes& xin, int n,
                        const int32_t* gather_src, const UnitTables& units, const ActPlanes& act, hipStream_t st,
                        hipEvent_t k_start = nullptr, hipEvent_t k_stop = nullptr);
void set_prefill_variant(int v);
int launch_down_mfma(const ferrite_moe_shape& s, const uint8_t* packed, const ActPlanes& act, int n,
                     const UnitTables& units, void* y, int y_dtype, hipStream_t st);

// block_ops.hip
int launch_rmsnorm(const float* x, const float* w, float eps, float* out, int n, int dim, hipStream_t st);
int launch_hc_post(const float* x, const float* residual, const float* post, const float* comb, float* out, int s,
                   int nh, int h, hipStream_t st);

// formats.hip
// q2 / scale2 (both or neither): the second term of a two-term quantisation, from the residual of the first.
int launch_act_quant(const void* x, int x_dtype, int64_t rows, int cols, uint8_t* q, uint8_t* scale, uint8_t* q2,
                     uint8_t* scale2, int operand_order, hipStream_t st);

}  // namespace fe
