/*
 * ferrite_hip.h -- C ABI of libferrite_hip.so: the MoE FFN layer of ferrite on one MI355X (gfx950).
 *
 * This is what a `HipBackend` in crates/ferrite-kernel would bind through dlopen, in the same way the
 * reference's CudaBackend binds libferrite_kernels.so (crates/ferrite-kernel/src/cuda.rs:24-400,5339-5427).
 * Conventions, all taken from that boundary:
 *   - every pointer is a DEVICE pointer unless its name ends in _host;
 *   - entry points return 0 on success and a non-zero FERRITE_* code otherwise (cuda.rs:411-425 maps
 *     non-zero to FerriteError::InvalidArg); FERRITE_DECLINED means "this shape is outside the kernel's
 *     contract, use another path" (kernels/cuda/dsv41_moe_align.cu:50-52);
 *   - launchers never allocate, never synchronise and never read the environment, so any of them may be
 *     recorded into a stream capture (cuda.rs:3008-3011); all scratch memory comes from the caller.  Kernels that
 *     use more than 64 KiB of LDS need a one-time function attribute per device: ferrite_hip_warmup() sets all of
 *     them, so that a first call inside a capture makes no runtime call besides its launches;
 *   - matrices are row-major, weights are [out_features, in_features] and ops compute x . w^T
 *     (crates/ferrite-kernel/src/lib.rs:61-66);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 */
#ifndef FERRITE_HIP_H
#define FERRITE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FERRITE_OK 0
#define FERRITE_ERR_INVALID_ARG 1  /* FerriteError::InvalidArg / ShapeMismatch */
#define FERRITE_DECLINED 2         /* shape outside this kernel's contract */
#define FERRITE_ERR_WORKSPACE 3    /* workspace too small */
#define FERRITE_ERR_RUNTIME 4      /* a HIP runtime call failed: see ferrite_hip_last_error() */

#define FERRITE_ABI_VERSION 3u

/* dtype tags for activation buffers (ferrite-types DType, crates/ferrite-types/src/lib.rs:16-25) */
#define FERRITE_DT_F32 0
#define FERRITE_DT_BF16 1

/* layer arithmetic modes */
#define FERRITE_MODE_F32_CHECK 0   /* f32 activations, weights dequantised exactly, f32 FMA dot products */
#define FERRITE_MODE_MFMA_FP8 1    /* activations quantised e4m3 per 32 (e8m0 scale), block-scaled MFMA */
#define FERRITE_MODE_MFMA_FP8_X2 2 /* the same with two-term activations: x ~ q1*s1 + q2*s2, the second term being the
                                    * e4m3-per-32 quantisation of what the first leaves over (about 8 significant
                                    * bits, bf16-class).  For decode-sized batches (n*topk < 16*n_experts) the
                                    * matrix cores idle behind the weight stream and the second term is nearly free;
                                    * prefill-sized batches are bound by the matrix cores and pay for it (64-row
                                    * units, twice the MFMAs per row: about 1.6 times the one-term layer). */

typedef void* ferrite_stream_t;

/* ---- identity: ferrite_kernels.cu:50-52, checked right after dlopen (cuda.rs:2061-2102) ---- */
const char* ferrite_kernel_build_id(void);
unsigned ferrite_kernel_abi_version(void);
/* Text of the last HIP runtime error seen by this thread ("" if none). */
const char* ferrite_hip_last_error(void);

/* Once per device, with that device current and outside any stream capture: raises the LDS limit of every kernel
 * that may need it (the reference warms its pools before a capture for the same reason, cuda.rs:627-657).
 * Optional for eager use: a launcher that finds its limit too low raises it on the spot. */
int ferrite_hip_warmup(void);

/* Process-wide test hooks (the reference's counterparts are environment gates read once into a OnceLock,
 * cuda.rs:5730-5731; here nothing reads the environment).  They change how a layer call tiles its work, and with it
 * the workspace layout: set them before sizing a workspace, not between sizing and use.
 *   FERRITE_OVERRIDE_UNIT_ROWS  0 = automatic (default), 16 = force the 16-row streaming kernels, 128 = force the
 *                               tiled kernels (units of 128 rows, or of 64 rows with two-term activations)
 *   FERRITE_OVERRIDE_Y_F32      1 = keep the expert outputs `y` in f32 on the tiled path (default 0: bf16)
 *   FERRITE_OVERRIDE_PREFILL_TILE  main loop of the 128-row units: 0 = default (gate/up: weights streamed into
 *                               registers by blocks of 8 waves; down: both operands staged through LDS), 1 = staged
 *                               for both GEMMs, 2 / 3 = streamed by blocks of 8 / 4 waves for both (same bits)
 *   FERRITE_OVERRIDE_HEAD       1 = router GEMM, routing, permutation and quantisation as separate launches whatever
 *                               the batch size (default 0: one fused launch for up to 256 tokens)  */
#define FERRITE_OVERRIDE_UNIT_ROWS 0
#define FERRITE_OVERRIDE_Y_F32 1
#define FERRITE_OVERRIDE_PREFILL_TILE 2
#define FERRITE_OVERRIDE_HEAD 3
int ferrite_hip_set_override(int which, int value);

/* ---- KernelBackend ops on the path (f32 device buffers, like the reference's GLM ABI) ---- */

/* KernelBackend::matmul (lib.rs:73; cpu.rs:82-122): out[n,o] = x[n,k] . w[o,k]^T (+ bias[o], may be NULL).
 * Each output is the reference's sequential-k f32 chain (separate multiply and add), bit for bit. */
int ferrite_matmul_f32(const float* x, const float* w, const float* bias, float* out, int n, int k, int o,
                       ferrite_stream_t stream);

/* KernelBackend::swiglu_limited (lib.rs:83-85; cpu.rs:178-203): gate_up [n, 2*inter] gate first. */
int ferrite_swiglu_limited_f32(const float* gate_up, float limit, float* out, int n, int inter,
                               ferrite_stream_t stream);

/* KernelBackend::moe_route (lib.rs:194-206; cpu.rs:528-572) extended with group-limited selection
 * (n_group = 1 is the reference's router).  probs [n,topk]; ids_f32 [n,topk] (the reference ABI stores ids
 * as f32) and/or ids_i32 [n,topk]; either ids pointer may be NULL.  Requires e <= 512, topk <= 32,
 * e % n_group == 0, topk <= topk_group * e / n_group.
 * NaN scores: CpuBackend panics on them (cpu.rs:560); this op follows the reference's device router instead
 * (kernels/cuda/ferrite_kernels.cu:1233-1270): a NaN score is never selected, and a slot that no finite score
 * can fill gets id -1 and weight 0 (it then drops out of the permutation and contributes nothing). */
int ferrite_moe_route(const float* logits, const float* bias, int n, int e, int topk, int n_group,
                      int topk_group, float routed_scaling, float* probs, float* ids_f32, int32_t* ids_i32,
                      ferrite_stream_t stream);

/* Token permutation by expert (kernels/cuda/dsv41_route.cu:194-315 contract; host golden
 * crates/ferrite-models/src/dsv41/chain_dev.rs:862-899): grouped order = expert ascending, then flat
 * assignment index i = t*topk + j ascending.  ids [n,topk] i32; a token may list an expert more than once (the
 * reference's vector chain_dev.rs:25042-25061 does): such assignments keep their slot order.  ids outside
 * [0, n_experts) drop out (perm_map = -1).  Outputs: counts[E], starts[E+1], perm_map[n*topk] (original ->
 * grouped), gather_src[n*topk] (grouped -> original, -1 past the end), active[E] (ascending experts with
 * counts > 0, -1 padded), n_active[1].  scratch: ferrite_moe_permute_scratch_bytes(n, topk, n_experts) bytes. */
size_t ferrite_moe_permute_scratch_bytes(int n, int topk, int n_experts);
int ferrite_moe_permute(const int32_t* ids, int n, int topk, int n_experts, int32_t* counts, int32_t* starts,
                        int32_t* perm_map, int32_t* gather_src, int32_t* active, int32_t* n_active,
                        void* scratch, size_t scratch_bytes, ferrite_stream_t stream);

/* MXFP4 -> f32 (crates/ferrite-models/src/dsv41/quant.rs:260-278): w [rows, cols/2] u8 (low nibble = even
 * column), scale [rows, cols/32] e8m0 -> dst [rows, cols] f32, exact. */
int ferrite_mxfp4_dequant(const uint8_t* w, const uint8_t* scale, int64_t rows, int64_t cols, float* dst,
                          ferrite_stream_t stream);

/* f32 / bf16 -> MXFP4 (quant.rs:217-238 act_quant_fp4 with block 32 and the power-of-two scale of :190-198):
 * x [rows, cols] -> codes [rows, cols/2] u8 (low nibble = even column), scale [rows, cols/32] e8m0 bytes.
 * For checkpoints that keep their experts unquantised (crates/ferrite-model/src/weights.rs:133-149). */
int ferrite_mxfp4_quant(const void* x, int x_dtype, int64_t rows, int64_t cols, uint8_t* codes, uint8_t* scale,
                        ferrite_stream_t stream);

/* Activation quantisation (quant.rs:190-214, block 32, power-of-two scale): x [rows, cols] (f32 or bf16) ->
 * q [rows, cols] e4m3 codes, scale [rows, cols/32] e8m0 bytes (2^(b-127)). */
int ferrite_act_quant_fp8(const void* x, int x_dtype, int64_t rows, int cols, uint8_t* q, uint8_t* scale,
                          ferrite_stream_t stream);

/* The two-term form of ferrite_act_quant_fp8 that FERRITE_MODE_MFMA_FP8_X2 feeds the matrix cores with: q1 / scale1
 * as above, then q2 / scale2 = the same quantiser applied to the residual x - decode(q1) * scale1 (one f32
 * multiply by the power-of-two scale and one f32 subtraction per value).  The reference's e4m3 path quantises
 * once (dsv41_quant_fp8, crates/ferrite-models/src/dsv41/kernels.rs:97-108); the decomposition itself is the one
 * it applies to its e2m1 activations: out = x - dequant(q) * scale in f32, quantised again, both terms run
 * against the same weight bytes (dsv41_sub_dequant_fp4, kernels/cuda/dsv41_kernels.cu:4138-4186). */
int ferrite_act_quant_fp8_x2(const void* x, int x_dtype, int64_t rows, int cols, uint8_t* q1, uint8_t* scale1,
                             uint8_t* q2, uint8_t* scale2, ferrite_stream_t stream);

/* ---- the fused layer: the counterpart of CudaBackend::moe_layer_dev (cuda.rs:5604-6142) for MXFP4 experts
 *      with group-limited routing; caller = Engine::moe_ffn (crates/ferrite-exec/src/lib.rs:1083-1166) ---- */

typedef struct ferrite_moe_shape {
    int hidden;        /* H, multiple of 128 */
    int n_experts;     /* E routed experts */
    int topk;          /* k */
    int inter;         /* I  = moe_intermediate, multiple of 128 */
    int shared_inter;  /* Is = shared expert intermediate (0 = none), multiple of 128 */
    int n_group;       /* 1 = ungrouped */
    int topk_group;
    float routed_scaling;
    float swiglu_limit;
} ferrite_moe_shape;

/* Checkpoint-layout MXFP4 weights (crates/ferrite-models/src/dsv41/weights.rs:340-341): codes
 * [E, rows, cols/2] u8 and e8m0 scales [E, rows, cols/32] u8, experts stacked contiguously. */
typedef struct ferrite_moe_weights {
    const float* router_w;     /* [E, H] f32 */
    const float* router_bias;  /* [E] f32 or NULL (zeros) */
    const uint8_t *gate_w, *gate_s; /* [E, I, H/2], [E, I, H/32] */
    const uint8_t *up_w, *up_s;
    const uint8_t *down_w, *down_s; /* [E, H, I/2], [E, H, I/32] */
    const uint8_t *sh_gate_w, *sh_gate_s, *sh_up_w, *sh_up_s; /* [Is, H/2], [Is, H/32] */
    const uint8_t *sh_down_w, *sh_down_s;                     /* [H, Is/2], [H, Is/32] */
} ferrite_moe_weights;

/* One-time repack of the checkpoint layout into the tile order the MFMA kernels stream (a pure permutation
 * of bytes; the reference does the analogous gate/up interleave at load time,
 * kernels/cuda/dsv41_experts_mxf4.cu:3430).  `packed` must hold ferrite_moe_packed_bytes(shape) bytes. */
size_t ferrite_moe_packed_bytes(const ferrite_moe_shape* shape);
int ferrite_moe_pack_weights(const ferrite_moe_shape* shape, const ferrite_moe_weights* w, uint8_t* packed,
                             ferrite_stream_t stream);
/* The same repack one expert at a time, for a loader that walks a checkpoint whose experts are separate tensors
 * (`{layer}.ffn.experts.{e}.w1|w2|w3.{weight,scale}`, crates/ferrite-models/src/dsv41/weights.rs:336-341) and
 * stages them one by one: `expert` in [0, n_experts), or n_experts for the shared expert.  gate/up (w1/w3) go
 * together, down (w2) on its own; either group may be left NULL.  The scale pitches are bytes between scale rows
 * of the source, 0 = dense (cols/32): a loader that pads scale rows (weights.rs:599 sf_plane_pitch, the fix for the
 * 10-byte w2 rows of kernels/cuda/dsv41_experts_mxf4.cu:121-168) passes its padded pitch; the packed layout itself
 * has no row pitch, its scales sit in operand order.  Sources are device-accessible memory, codes 16-byte aligned. */
typedef struct ferrite_moe_expert_src {
    const uint8_t *gate_w, *gate_s, *up_w, *up_s; /* [I, H/2], [I, pitch] */
    const uint8_t *down_w, *down_s;               /* [H, I/2], [H, pitch] */
    int64_t gate_up_scale_pitch, down_scale_pitch;
} ferrite_moe_expert_src;
int ferrite_moe_pack_expert(const ferrite_moe_shape* shape, int expert, const ferrite_moe_expert_src* src,
                            uint8_t* packed, ferrite_stream_t stream);
/* The router's part of the packed buffer (the k-blocked transpose of router_w [E, H] f32). */
int ferrite_moe_pack_router(const ferrite_moe_shape* shape, const float* router_w, uint8_t* packed,
                            ferrite_stream_t stream);

/* Inverse view for verification: dequantise matrix `which` (0 gate, 1 up, 2 down) of expert `expert`
 * (expert == n_experts selects the shared expert) from the packed buffer to f32 [rows, cols]. */
int ferrite_moe_packed_dequant(const ferrite_moe_shape* shape, const uint8_t* packed, int expert, int which,
                               float* dst, ferrite_stream_t stream);

/* Pointers into the caller's workspace where the layer leaves its intermediates (for tests / tracing). */
typedef struct ferrite_moe_workspace_view {
    float* logits;       /* [n, E] */
    float* probs;        /* [n, topk] */
    float* ids_f32;      /* [n, topk] */
    int32_t* ids;        /* [n, topk] */
    int32_t* counts;     /* [E] */
    int32_t* starts;     /* [E+1] */
    int32_t* perm_map;   /* [n*topk] */
    int32_t* gather_src; /* [n*topk] */
    int32_t* active;     /* [E] */
    int32_t* n_active;   /* [1] */
    float* y;            /* [(n*topk + n), H] expert outputs in grouped order, then the shared expert's rows; f32,
                          * except bf16 (same shape, half the bytes) when ferrite_moe_layer_unit_rows() is 64 or
                          * 128 and the FERRITE_OVERRIDE_Y_F32 override is off */
} ferrite_moe_workspace_view;

/* What a layer call with these arguments would answer before it enqueues anything: FERRITE_OK, or
 * FERRITE_DECLINED (this batch size / shape is outside this mode's contract: the caller falls back to another mode,
 * as CudaBackend does when a fused kernel declines, cuda.rs:5763-5765,5940,5990 - the order is two-term MFMA,
 * one-term MFMA, f32; the MFMA modes decline hidden / intermediate sizes that are not multiples of 128), or
 * FERRITE_ERR_INVALID_ARG.  A declined mode has no workspace size either (ferrite_moe_layer_workspace_bytes is 0). */
int ferrite_moe_layer_check(const ferrite_moe_shape* shape, int n, int mode);
size_t ferrite_moe_layer_workspace_bytes(const ferrite_moe_shape* shape, int n, int mode);
/* Rows per unit (the token tile of the expert GEMMs) a layer call with these arguments uses: 16 = weights streamed
 * once per unit (decode-sized batches: n*topk < 16*n_experts, any activation format); beyond that the tiled kernels,
 * 128 = one-term activations, 64 = two-term activations (both planes of 64 rows fill the same tile); 0 for an
 * unsupported shape.  The choice is a pure function of (shape, n, mode) and of the FERRITE_OVERRIDE_UNIT_ROWS
 * override, like the workspace layout that depends on it.
 * No counterpart in the reference, whose grouped GEMM has one tile shape (dsv41_moe.cu); informational. */
int ferrite_moe_layer_unit_rows(const ferrite_moe_shape* shape, int n, int mode);
/* Must run once on a freshly allocated workspace before its first layer call (it clears the arrival counters
 * the fused routing kernel keeps there; the kernel leaves them cleared, so replays need no further call).
 * Workspaces are owned by the caller like every other buffer (DevBuf pool, cuda.rs:558-744). */
int ferrite_moe_layer_workspace_init(const ferrite_moe_shape* shape, int n, int mode, void* workspace,
                                     size_t workspace_bytes, ferrite_stream_t stream);
int ferrite_moe_layer_workspace_view(const ferrite_moe_shape* shape, int n, int mode, void* workspace,
                                     ferrite_moe_workspace_view* view_host);

/* The layer.  x [n, H] (x_dtype), out [n, H] (out_dtype).  mode FERRITE_MODE_F32_CHECK reads `w` (checkpoint
 * layout) and requires f32 x; the FERRITE_MODE_MFMA_* modes read `packed` and w->router_bias.  `packed` carries the
 * router weight, so w->router_w may be NULL with it; the few shapes whose router falls back to the checkpoint
 * layout (very large hidden) then return FERRITE_ERR_INVALID_ARG.  n > 65535 and routing parameters outside
 * ferrite_moe_route's limits are refused up front (FERRITE_DECLINED / FERRITE_ERR_INVALID_ARG, as that op returns
 * them), before anything is enqueued.
 * The launch sequence depends only on (shape, n, mode), never on the routing, so a captured graph of it
 * replays correctly for any input (the GraphCapable contract, crates/ferrite-kernel/src/graph.rs:48-64). */
int ferrite_moe_layer_mxfp4(const ferrite_moe_shape* shape, const ferrite_moe_weights* w, const uint8_t* packed,
                            const void* x, int x_dtype, int n, void* out, int out_dtype, int mode,
                            void* workspace, size_t workspace_bytes, ferrite_stream_t stream);

/* The same layer for callers that cannot allocate device memory at all and so have no workspace to pass: code
 * under a stream capture that arrives without buffers, tight serving loops, harnesses that forbid hipMalloc.  It has
 * no counterpart in the reference.  The workspace is an
 * array of FERRITE_STATIC_WORKSPACE_BYTES built into the library (each GPU the library runs on holds one copy until
 * the process ends); inputs, weights and outputs are still the caller's.  Same results as ferrite_moe_layer_mxfp4,
 * bit for bit.  Calls whose workspace (ferrite_moe_layer_workspace_bytes) exceeds the array return
 * FERRITE_ERR_WORKSPACE with the two sizes in ferrite_hip_last_error(); at H 4096, top-8, I 1536 that is up to
 * about 100 tokens.  It calls no hipMalloc / hipFree or anything else that allocates, and does not synchronise; the
 * first call on a device looks the array's address up (ferrite_hip_warmup() does that ahead of time, e.g. before a
 * capture).  Every call on a GPU uses that GPU's one array: calls that overlap on the same GPU (two streams, two
 * threads) race, and the workspace-view entry points do not apply. */
#define FERRITE_STATIC_WORKSPACE_BYTES (16u << 20)
int ferrite_moe_layer_mxfp4_static(const ferrite_moe_shape* shape, const ferrite_moe_weights* w, const uint8_t* packed,
                                   const void* x, int x_dtype, int n, void* out, int out_dtype, int mode,
                                   ferrite_stream_t stream);

/* ---- the steps on either side of the layer (crates/ferrite-exec/src/lib.rs:487-492) ---- */

/* KernelBackend::rmsnorm (crates/ferrite-kernel/src/lib.rs:76; CpuBackend, cpu.rs:124-143; CUDA: ferrite_rmsnorm,
 * cuda.rs): x, out [n, dim] f32, w [dim] f32.  Bit-exact to the reference: the squares of a row are summed left to
 * right in f32, inv = 1 / sqrt(ss / dim + eps), out = (x * inv) * w. */
int ferrite_rmsnorm_f32(const float* x, const float* w, float eps, float* out, int n, int dim, ferrite_stream_t stream);

/* KernelBackend::hc_post (lib.rs:256; cpu.rs:788-807; CUDA hc_post_kernel, kernels/cuda/ferrite_kernels.cu:2679):
 * out[t,i,:] = post[t,i] * x[t,:] + sum_k comb[t,k,i] * residual[t,k,:] in k order, bit-exact.
 * x [s,h], residual [s,nh,h], post [s,nh], comb [s,nh,nh], out [s,nh,h], all f32; nh <= 8, h % 4 == 0, 16-byte
 * aligned x/residual/out, else FERRITE_DECLINED / FERRITE_ERR_INVALID_ARG. */
int ferrite_hc_post_f32(const float* x, const float* residual, const float* post, const float* comb, float* out,
                        int s, int nh, int h, ferrite_stream_t stream);

/* The FFN half of a decoder layer in one call, the three statements of crates/ferrite-exec/src/lib.rs:487-492:
 *     hfn     = rmsnorm(li, post_attention_layernorm.weight, eps)
 *     ffn_out = moe_ffn(hfn)                       (ferrite_moe_layer_mxfp4 on f32 activations)
 *     out     = hc_post(ffn_out, residual, post, comb)
 * li [n, H] f32 (the mixed stream that hc_pre produced), out [n, nh, H] f32.  With residual == NULL the call ends
 * after the second statement and out is ffn_out [n, H] (post, comb and nh are then ignored): the pre-norm layer
 * without hyper-connections, which is also how consecutive layers are chained (out of one = li of the next).  The workspace is the layer's followed by
 * two [n, H] f32 buffers: size it with ferrite_moe_block_workspace_bytes and initialise it once with
 * ferrite_moe_layer_workspace_init (which only touches the layer's part).  Same rules as the layer call: no
 * allocation, no synchronisation, a launch sequence that depends only on (shape, n, mode), capturable.
 * Aliasing: out may be the residual buffer itself (the streams updated in place: every thread reads its columns of
 * all nh streams before it writes any), but must not overlap it in any other way, and must not overlap li. */
typedef struct {
    const float* norm_w;    /* [H] */
    float eps;
    const float* residual;  /* [n, nh, H], or NULL: no hc_post */
    const float* post;      /* [n, nh] */
    const float* comb;      /* [n, nh, nh] */
    int nh;                 /* hyper-connection streams (hc_mult), <= 8 */
} ferrite_moe_block_args;

size_t ferrite_moe_block_workspace_bytes(const ferrite_moe_shape* shape, int n, int mode);
int ferrite_moe_block_mxfp4(const ferrite_moe_shape* shape, const ferrite_moe_weights* w, const uint8_t* packed,
                            const float* li, const ferrite_moe_block_args* blk, int n, float* out, int mode,
                            void* workspace, size_t workspace_bytes, ferrite_stream_t stream);

/* The same layer with HIP events recorded on `stream` at the stage boundaries, the counterpart of the
 * reference's FERRITE_TIMING probes (crates/ferrite-exec/src/lib.rs:1184-1299).  stage_events_host is a host
 * array of FERRITE_MOE_STAGE_EVENTS hipEvent_t handles (any may be NULL): [0] before the router GEMM, then
 * after: [1] router GEMM, [2] routing, [3] permutation, [4] activation quantisation (== [3] in f32 mode),
 * [5] gate/up GEMM + SwiGLU, [6] down GEMM, [7] combine; [8] and [9] bracket the gate/up kernel itself on the
 * device (start and end of its execution, without the launch gap that [4]..[5] includes; MFMA mode only).
 * Not capturable. */
#define FERRITE_MOE_STAGE_EVENTS 10
int ferrite_moe_layer_mxfp4_timed(const ferrite_moe_shape* shape, const ferrite_moe_weights* w,
                                  const uint8_t* packed, const void* x, int x_dtype, int n, void* out,
                                  int out_dtype, int mode, void* workspace, size_t workspace_bytes,
                                  ferrite_stream_t stream, void* const* stage_events_host);

/* ---- graph capture: ferrite_graph_begin/end/instantiate/launch (cuda.rs:284-287) ---- */
int ferrite_graph_begin(ferrite_stream_t stream);
int ferrite_graph_end(ferrite_stream_t stream, void** graph_exec_out);
int ferrite_graph_launch(void* graph_exec, ferrite_stream_t stream);
int ferrite_graph_destroy(void* graph_exec);

#ifdef __cplusplus
}
#endif
#endif
