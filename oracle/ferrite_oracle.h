/*
 * ferrite_oracle.h -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C, CPU restatement of ferrite's f32 golden path for the MoE FFN layer
 * (CpuBackend + Engine::moe_ffn) and of the dsv41 MXFP4 / e4m3 / ue8m0 format
 * primitives.  It exists to check the HIP library and to provide the "CPU port"
 * timing baseline.  Nothing in the shipped library or package may include, link
 * or call it: only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg.
 *
 * Every function cites the reference file:line it follows (paths relative to the
 * reference checkout).  Arithmetic order is the reference's: sequential-k f32
 * dot products with a separate multiply and add (build with -ffp-contract=off,
 * no fast-math), libm expf for sigmoid / silu.
 *
 * Pinning status (what fixes each function besides this restatement):
 *   formats (e2m1/e4m3/ue8m0/fast_*, act_quant_fp8, dequant_fp4_row32)
 *       -> known-answer tests of crates/ferrite-models/src/dsv41/quant.rs:336-501,
 *          exhaustive code sweeps, torch.float8_e4m3fn casts.            PINNED
 *   fo_matmul / fo_swiglu_limited / fo_moe_route
 *       -> crates/ferrite-kernel/tests/golden.rs:14-27,44-55,189-210,
 *          gpu_smoke.rs:139-155 ramp fixture (closed form), brute force. PINNED
 *   fo_rmsnorm / fo_hc_post (the steps before and after the layer)
 *       -> golden.rs:30-42 closed form; no numeric vector for hc_post exists in the reference
 *          (gpu_smoke.rs:308-348 compares device against CpuBackend), so it is pinned by a NumPy
 *          statement with explicit f32 rounding, the identity-mix special case and linearity.  PINNED
 *   fo_moe_permute / fo_moe_align_host
 *       -> chain_dev.rs:25042-25061 vector, stable-sort closed form.     PINNED
 *   fo_moe_ffn_mxfp4 (f32 mode)
 *       -> gpu_smoke.rs:437-562 small layer fixture re-derived in float64
 *          NumPy, dsv41 ops.rs:1100-1105 clamp convention.               PINNED
 *   fo_moe_route_grouped (n_group / topk_group)
 *       -> NO reference implementation or vector exists.  PARITY UNPINNED.
 *          Checked only by reduction to fo_moe_route (n_group==1 or
 *          topk_group==n_group) and brute force over group subsets.
 */
#ifndef FERRITE_ORACLE_H
#define FERRITE_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- formats: crates/ferrite-models/src/dsv41/quant.rs ---- */
float   fo_e2m1_decode(uint8_t code);                 /* quant.rs:22-35   */
uint8_t fo_e2m1_encode(float x);                      /* quant.rs:40-55   */
float   fo_e4m3_decode(uint8_t b);                    /* quant.rs:84-93   */
uint8_t fo_e4m3_encode(float x);                      /* quant.rs:98-124  */
float   fo_ue8m0_decode(uint8_t b);                   /* quant.rs:130-136 */
uint8_t fo_ue8m0_encode_pow2(int exp);                /* quant.rs:138-140 */
int     fo_fast_log2_ceil(float x);                   /* quant.rs:155-160 */
float   fo_fast_pow2(int e);                          /* quant.rs:163-165 */
float   fo_fast_round_scale(float amax);              /* quant.rs:169-174 */
/* quant.rs:190-214: y[len] e4m3 codes, s[len/block] scales */
void    fo_act_quant_fp8(const float* x, size_t len, int block, int round_scale, uint8_t* y, float* s);
/* Two-term form (no reference counterpart: its quantiser composed with one f32 subtraction): q1/s1 =
 * act_quant_fp8(x, 32, round_scale), q2/s2 = act_quant_fp8(x - decode(q1)*s1, 32, round_scale).
 * PARITY UNPINNED by the reference; pinned by construction from fo_act_quant_fp8 (a NumPy composition in the tests). */
void    fo_act_quant_fp8_x2(const float* x, size_t len, uint8_t* q1, float* s1, uint8_t* q2, float* s2);
/* quant.rs:217-238: packed[len/2], s[len/block] */
void    fo_act_quant_fp4(const float* x, size_t len, int block, int round_scale, uint8_t* packed, float* s);
/* quant.rs:260-278: w [out, inn/2] u8, scale [out, inn/32] u8 -> dst [out, inn] f32 */
void    fo_dequant_fp4_row32(const uint8_t* w, const uint8_t* scale, size_t out, size_t inn, float* dst);

/* ---- CpuBackend ops: crates/ferrite-kernel/src/cpu.rs ---- */
/* cpu.rs:82-122. out[n,o] = x[n,k] . w[o,k]^T (+bias[o]); returns 0, or 1 on bad dims */
int fo_matmul(const float* x, const float* w, const float* bias, float* out, int n, int k, int o);
/* cpu.rs:178-203. gate_up [n, 2*inter] (gate first), out [n, inter] */
int fo_swiglu_limited(const float* gate_up, float limit, float* out, int n, int inter);
/* cpu.rs:124-143 */
int fo_rmsnorm(const float* x, const float* w, float eps, float* out, int n, int dim);
/* cpu.rs:788-807: x [s,h], residual [s,nh,h], post [s,nh], comb [s,nh,nh], out [s,nh,h] */
int fo_hc_post(const float* x, const float* residual, const float* post, const float* comb, float* out, int s, int nh,
               int h);
/* cpu.rs:528-572. probs/ids [n, topk]; ids as f32 like the reference. 2 = NaN score (reference panics) */
int fo_moe_route(const float* logits, const float* bias, int n, int e, int topk, float routed_scaling,
                 float* probs, float* ids);
/* Group-limited variant (no reference counterpart; see header comment). */
int fo_moe_route_grouped(const float* logits, const float* bias, int n, int e, int topk, int n_group,
                         int topk_group, float routed_scaling, float* probs, float* ids);
/* The same with the treatment of NaN scores as a parameter: 0 = error 2, as above (CpuBackend panics, cpu.rs:560);
 * 1 = the reference's device router (kernels/cuda/ferrite_kernels.cu:1233-1270): never selected, unfillable slots
 * get id -1 and weight 0.  Pinned by its special cases only (no NaN: equal to the above; all NaN: all -1). */
int fo_moe_route_grouped_nan(const float* logits, const float* bias, int n, int e, int topk, int n_group,
                             int topk_group, float routed_scaling, int nan_policy, float* probs, float* ids);
/* cpu.rs:574-625 */
int fo_expert_ffn(const float* x, const float* gate_w, const float* up_w, const float* down_w, float limit,
                  float* out, int m, int hidden, int inter);

/* ---- permutation: kernels/cuda/dsv41_route.cu:194-315 ---- */
/* ids [n*topk] i32. counts[E], starts[E+1], perm_map[n*topk], gather_src[n*topk], active[E], n_active[1] */
int fo_moe_permute(const int32_t* ids, int n, int topk, int n_experts, int32_t* counts, int32_t* starts,
                   int32_t* perm_map, int32_t* gather_src, int32_t* active, int32_t* n_active);
/* crates/ferrite-models/src/dsv41/chain_dev.rs:862-899. order[seg_cap*bm], counts[seg_cap], eid[seg_cap];
 * returns nseg >= 0, or -1 for "None" (declined). */
int fo_moe_align_host(const int32_t* idx, int len, int topk, int seg_cap, int bm, int32_t* order,
                      int32_t* counts, int32_t* eid);

/* ---- the layer: crates/ferrite-exec/src/lib.rs:1083-1166,1316-1332 ---- */
typedef struct {
    int n;               /* tokens */
    int hidden;          /* H */
    int n_experts;       /* E routed */
    int topk;            /* k */
    int inter;           /* I  (routed moe_intermediate) */
    int shared_inter;    /* Is (0 = no shared expert) */
    int n_group;         /* 1 = ungrouped (the reference's router) */
    int topk_group;
    float routed_scaling;
    float swiglu_limit;
    int act_mode;        /* 0: f32 activations (CpuBackend proper);
                            1: x and the SwiGLU output are passed through act_quant_fp8(block 32,
                               round_scale) and dequantised before each expert GEMM (quant.rs:201-214), where the
                               reference's device chain quantises (dsv41_quant_fp8 in front of the first GEMM,
                               dsv41_swiglu_limit_q after the SwiGLU: kernels.rs:97-108,586-598);
                            2: the same two places through the two-term quantiser (fo_act_quant_fp8_x2) */
    int n_threads;       /* 1 = faithful single thread; >1 OpenMP over tokens/rows (never over k) */
} fo_moe_cfg;

typedef struct {
    /* routed experts, checkpoint layout (dsv41/weights.rs:340-341): codes [E, rows, cols/2], scales [E, rows, cols/32] */
    const uint8_t *gate_w, *gate_s;   /* [E, I, H/2], [E, I, H/32] */
    const uint8_t *up_w, *up_s;
    const uint8_t *down_w, *down_s;   /* [E, H, I/2], [E, H, I/32] */
    const uint8_t *sh_gate_w, *sh_gate_s, *sh_up_w, *sh_up_s, *sh_down_w, *sh_down_s; /* Is rows/cols */
    const float* router_w;            /* [E, H] f32 */
    const float* router_bias;         /* [E] f32 or NULL (zeros) */
} fo_moe_weights;

/* x [n,H] f32.  tok_sel/n_sel: the tokens whose expert FFN + combine are evaluated (NULL = all);
 * routing is always evaluated for every token.  Outputs (any may be NULL): out [n_sel or n, H]
 * (row r = token tok_sel[r]), logits [n,E], probs/ids [n,topk] (ids f32).  Returns 0 on success. */
int fo_moe_ffn_mxfp4(const fo_moe_cfg* cfg, const fo_moe_weights* w, const float* x, const int32_t* tok_sel,
                     int n_sel, float* out, float* logits, float* probs, float* ids);

#ifdef __cplusplus
}
#endif
#endif
