/*
 * ferrite_oracle.c -- TEST INFRASTRUCTURE ONLY (see ferrite_oracle.h).
 *
 * CPU restatement of the reference's f32 MoE FFN path.  Build:
 *   gcc -O2 -std=c11 -fPIC -shared -fopenmp -ffp-contract=off -fno-fast-math \
 *       -o libferrite_oracle.so ferrite_oracle.c -lm
 * -ffp-contract=off matters: the reference's dot products are a separate f32
 * multiply and add per element (crates/ferrite-kernel/src/cpu.rs:106-111).
 */
#include "ferrite_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ formats */

/* quant.rs:22-25 FP4_TABLE */
static const float FO_FP4_TABLE[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                       0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};
#define FO_FP4_MAX 6.0f
#define FO_FP8_MAX 448.0f

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* quant.rs:176-178 exp2i: 2^e with the biased exponent clamped into [0, 254] */
static inline float exp2i(int e) {
    int b = e + 127;
    if (b < 0) b = 0;
    if (b > 254) b = 254;
    return u2f((uint32_t)b << 23);
}

float fo_e2m1_decode(uint8_t code) { return FO_FP4_TABLE[code & 0xF]; }

/* quant.rs:40-55: nearest magnitude, first (lowest slot) wins ties, sign bit 8 when x < 0 */
uint8_t fo_e2m1_encode(float x) {
    static const float mag[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
    float a = fabsf(x);
    if (a > FO_FP4_MAX) a = FO_FP4_MAX; /* f32::min */
    int best = 0;
    float bestd = INFINITY;
    for (int i = 0; i < 8; ++i) {
        float d = fabsf(a - mag[i]);
        if (d < bestd) { bestd = d; best = i; }
    }
    return (uint8_t)(best | (x < 0.0f ? 8 : 0));
}

/* quant.rs:84-93 */
float fo_e4m3_decode(uint8_t b) {
    float sign = (b & 0x80) ? -1.0f : 1.0f;
    int e = (b >> 3) & 0x0F;
    float m = (float)(b & 0x07);
    if (e == 0) return sign * m * (1.0f / 512.0f);
    return sign * (1.0f + m / 8.0f) * exp2i(e - 7);
}

/* f32::round_ties_even */
static inline float round_ties_even_f(float v) { return nearbyintf(v); /* default FE_TONEAREST */ }

/* quant.rs:98-124 */
uint8_t fo_e4m3_encode(float x) {
    uint8_t sign = signbit(x) ? 0x80 : 0;
    if (!isfinite(x)) return sign | 0x7E;
    float a = fabsf(x);
    if (a > FO_FP8_MAX) a = FO_FP8_MAX;
    if (a == 0.0f) return sign;
    if (a < exp2i(-6)) {
        float m = round_ties_even_f(a * 512.0f);
        if (m < 0.0f) m = 0.0f;
        if (m > 7.0f) m = 7.0f;
        return sign | (uint8_t)m;
    }
    int e = (int)((f2u(a) >> 23) & 0xFF) - 127;
    if (e > 8) e = 8;
    float m = ((a / exp2i(e)) - 1.0f) * 8.0f;
    int mi = (int)round_ties_even_f(m);
    if (mi >= 8) { mi = 0; e += 1; }
    if (e > 8) return sign | 0x7E;
    return sign | (uint8_t)((((uint8_t)(e + 7)) & 0x0F) << 3) | ((uint8_t)mi & 0x07);
}

/* quant.rs:130-136 */
float fo_ue8m0_decode(uint8_t b) { return b == 0xFF ? NAN : exp2i((int)b - 127); }

/* quant.rs:138-140 */
uint8_t fo_ue8m0_encode_pow2(int exp) {
    int v = exp + 127;
    if (v < 0) v = 0;
    if (v > 0xFE) v = 0xFE;
    return (uint8_t)v;
}

/* quant.rs:155-160 */
int fo_fast_log2_ceil(float x) {
    uint32_t bits = f2u(x);
    int ex = (int)((bits >> 23) & 0xFF);
    uint32_t man = bits & ((1u << 23) - 1);
    return ex - 127 + (man != 0 ? 1 : 0);
}

/* quant.rs:163-165 */
float fo_fast_pow2(int e) { return u2f((uint32_t)((e + 127) << 23)); }

/* quant.rs:169-174 */
float fo_fast_round_scale(float amax) {
    if (amax == 0.0f) return 0.0f;
    return fo_fast_pow2(fo_fast_log2_ceil(amax / FO_FP8_MAX));
}

/* quant.rs:190-198 block_scale */
static float block_scale(const float* x, int len, float maxv, int round_scale) {
    float amax = 0.0f;
    for (int i = 0; i < len; ++i) {
        float v = fabsf(x[i]);
        if (v > amax) amax = v; /* f32::max fold; NaN inputs are outside the contract */
    }
    float s = round_scale ? fo_fast_pow2(fo_fast_log2_ceil(amax / maxv)) : amax / maxv;
    if (!(s > FLT_MIN)) s = FLT_MIN; /* .max(f32::MIN_POSITIVE) */
    return s;
}

/* quant.rs:201-214 */
void fo_act_quant_fp8(const float* x, size_t len, int block, int round_scale, uint8_t* y, float* s) {
    size_t nb = len / (size_t)block;
    for (size_t b = 0; b < nb; ++b) {
        const float* blk = x + b * block;
        float sc = block_scale(blk, block, FO_FP8_MAX, round_scale);
        s[b] = sc;
        for (int i = 0; i < block; ++i) y[b * block + i] = fo_e4m3_encode(blk[i] / sc);
    }
}

/* quant.rs:217-238 */
void fo_act_quant_fp4(const float* x, size_t len, int block, int round_scale, uint8_t* packed, float* s) {
    size_t nb = len / (size_t)block;
    uint8_t* nib = (uint8_t*)malloc(len ? len : 1);
    for (size_t b = 0; b < nb; ++b) {
        const float* blk = x + b * block;
        float sc = block_scale(blk, block, FO_FP4_MAX, round_scale);
        s[b] = sc;
        for (int i = 0; i < block; ++i) nib[b * block + i] = fo_e2m1_encode(blk[i] / sc);
    }
    for (size_t i = 0; i < len / 2; ++i) packed[i] = (uint8_t)((nib[2 * i] & 0x0F) | ((nib[2 * i + 1] & 0x0F) << 4));
    free(nib);
}

/* quant.rs:260-278: low nibble = even column (quant.rs:57-68).  Same per-element arithmetic as the reference
 * (table[code] * 2^(scale-127)), walked one 32-column block at a time; rows are independent, so `nt` > 1
 * splits them over threads. */
static void dequant_fp4_row32_mt(const uint8_t* w, const uint8_t* scale, size_t out, size_t inn, float* dst, int nt) {
    const size_t nb_in = inn / 32;
#pragma omp parallel for num_threads(nt > 1 ? nt : 1) schedule(static)
    for (size_t r = 0; r < out; ++r) {
        const uint8_t* row = w + r * (inn / 2);
        float* d = dst + r * inn;
        for (size_t b = 0; b < nb_in; ++b) {
            float s = fo_ue8m0_decode(scale[r * nb_in + b]);
            for (size_t i = 0; i < 16; ++i) {
                uint8_t byte = row[b * 16 + i];
                d[b * 32 + 2 * i] = FO_FP4_TABLE[byte & 0x0F] * s;
                d[b * 32 + 2 * i + 1] = FO_FP4_TABLE[(byte >> 4) & 0x0F] * s;
            }
        }
    }
}

void fo_dequant_fp4_row32(const uint8_t* w, const uint8_t* scale, size_t out, size_t inn, float* dst) {
    dequant_fp4_row32_mt(w, scale, out, inn, dst, 1);
}

/* ------------------------------------------------------------- CpuBackend ops */

/* One output element: cpu.rs:106-111.  s = 0; for l: s += x[l]*w[l] (separate mul, add). */
static inline float dot_seq(const float* x, const float* w, int k) {
    float s = 0.0f;
    for (int l = 0; l < k; ++l) s += x[l] * w[l];
    return s;
}

/* Eight rows of w against one x, each with its own sequential chain: identical values to eight
 * dot_seq calls, but the independent chains pipeline. */
static inline void dot_seq8(const float* x, const float* w, size_t ldw, int k, float* out8) {
    float s0 = 0, s1 = 0, s2 = 0, s3 = 0, s4 = 0, s5 = 0, s6 = 0, s7 = 0;
    const float *w0 = w, *w1 = w + ldw, *w2 = w + 2 * ldw, *w3 = w + 3 * ldw, *w4 = w + 4 * ldw,
                *w5 = w + 5 * ldw, *w6 = w + 6 * ldw, *w7 = w + 7 * ldw;
    for (int l = 0; l < k; ++l) {
        float xv = x[l];
        s0 += xv * w0[l]; s1 += xv * w1[l]; s2 += xv * w2[l]; s3 += xv * w3[l];
        s4 += xv * w4[l]; s5 += xv * w5[l]; s6 += xv * w6[l]; s7 += xv * w7[l];
    }
    out8[0] = s0; out8[1] = s1; out8[2] = s2; out8[3] = s3; out8[4] = s4; out8[5] = s5; out8[6] = s6; out8[7] = s7;
}

/* x[k] against o rows of w -> out[o] */
static void gemv_seq(const float* x, const float* w, int k, int o, float* out) {
    int j = 0;
    for (; j + 8 <= o; j += 8) dot_seq8(x, w + (size_t)j * k, (size_t)k, k, out + j);
    for (; j < o; ++j) out[j] = dot_seq(x, w + (size_t)j * k, k);
}

/* cpu.rs:82-122 */
int fo_matmul(const float* x, const float* w, const float* bias, float* out, int n, int k, int o) {
    if (n < 0 || k < 0 || o < 0) return 1;
    for (int i = 0; i < n; ++i) {
        gemv_seq(x + (size_t)i * k, w, k, o, out + (size_t)i * o);
        if (bias)
            for (int j = 0; j < o; ++j) out[(size_t)i * o + j] += bias[j];
    }
    return 0;
}

/* cpu.rs:178-203 */
static inline float swiglu1(float g, float u, float limit) {
    float gi = g > limit ? limit : g;
    float ui = u;              /* f32::clamp(-limit, limit) */
    if (ui < -limit) ui = -limit;
    if (ui > limit) ui = limit;
    float silu = gi / (1.0f + expf(-gi));
    return silu * ui;
}

int fo_swiglu_limited(const float* gate_up, float limit, float* out, int n, int inter) {
    if (n < 0 || inter < 0) return 1;
    size_t two_i = (size_t)2 * inter;
    for (int i = 0; i < n; ++i)
        for (int j = 0; j < inter; ++j)
            out[(size_t)i * inter + j] = swiglu1(gate_up[i * two_i + j], gate_up[i * two_i + inter + j], limit);
    return 0;
}

/* crates/ferrite-kernel/src/cpu.rs:124-143 (KernelBackend::rmsnorm, lib.rs:76): per row, the squares are summed left to
 * right in f32 (Iterator::sum is a sequential fold; square and add are separately rounded), divided by the row length,
 * inv = 1 / sqrt(ss + eps) with correctly rounded sqrt and division, out = (x * inv) * w. */
int fo_rmsnorm(const float* x, const float* w, float eps, float* out, int n, int dim) {
    if (n < 0 || dim <= 0) return 1;
    for (int i = 0; i < n; ++i) {
        const float* row = x + (size_t)i * dim;
        float ss = 0.0f;
        for (int j = 0; j < dim; ++j) {
            float sq = row[j] * row[j];
            ss = ss + sq;
        }
        ss = ss / (float)dim;
        float inv = 1.0f / sqrtf(ss + eps);
        for (int j = 0; j < dim; ++j) {
            float t = row[j] * inv;
            out[(size_t)i * dim + j] = t * w[j];
        }
    }
    return 0;
}

/* crates/ferrite-kernel/src/cpu.rs:788-807 (KernelBackend::hc_post, lib.rs:256; same loop in
 * crates/ferrite-exec/src/mhc.rs:195-213): out[t,i,:] = post[t,i] * x[t,:] + sum_k comb[t,k,i] * residual[t,k,:],
 * accumulated in k order with separately rounded multiply and add.
 * x [s,h], residual [s,nh,h], post [s,nh], comb [s,nh,nh], out [s,nh,h]. */
int fo_hc_post(const float* x, const float* residual, const float* post, const float* comb, float* out, int s, int nh,
               int h) {
    if (s < 0 || nh <= 0 || h <= 0) return 1;
    for (int t = 0; t < s; ++t)
        for (int i = 0; i < nh; ++i)
            for (int j = 0; j < h; ++j) {
                float acc = post[(size_t)t * nh + i] * x[(size_t)t * h + j];
                for (int k = 0; k < nh; ++k) {
                    float p = comb[((size_t)t * nh + k) * nh + i] * residual[((size_t)t * nh + k) * h + j];
                    acc = acc + p;
                }
                out[((size_t)t * nh + i) * h + j] = acc;
            }
    return 0;
}

typedef struct { float s; int j; } scored_t;

/* cpu.rs:560: descending score, ties -> ascending index.  A strict total order, so any sort agrees
 * with the reference's stable sort. */
static int scored_cmp(const void* a, const void* b) {
    const scored_t* x = (const scored_t*)a;
    const scored_t* y = (const scored_t*)b;
    if (x->s > y->s) return -1;
    if (x->s < y->s) return 1;
    return (x->j > y->j) - (x->j < y->j);
}

/* one row of cpu.rs:546-569 given the candidate mask (NULL = all experts).
 * nan_policy 0: a NaN score is an error (partial_cmp().unwrap() panics in the reference);
 * nan_policy 1: the reference's device router (kernels/cuda/ferrite_kernels.cu:1233-1270): its arg-max
 *   comparisons are false for NaN, so a NaN score is never selected, and a slot that no finite score can fill
 *   gets id -1 and weight 0. */
static int route_row(const float* ls, const float* bs, int e, int topk, float scaling, const uint8_t* keep,
                     int nan_policy, float* sig, scored_t* scored, float* probs, float* ids) {
    int nc = 0;
    for (int j = 0; j < e; ++j) {
        sig[j] = 1.0f / (1.0f + expf(-ls[j]));
        float c = sig[j] + bs[j];
        if (isnan(c)) {
            if (nan_policy == 0) return 2;
            continue;
        }
        if (!keep || keep[j]) { scored[nc].s = c; scored[nc].j = j; ++nc; }
    }
    if (topk > nc && nan_policy == 0) return 1;
    qsort(scored, (size_t)nc, sizeof(scored_t), scored_cmp);
    const int nsel = topk < nc ? topk : nc;
    float sum = 0.0f;
    for (int r = 0; r < nsel; ++r) sum += sig[scored[r].j];
    for (int r = 0; r < nsel; ++r) {
        int j = scored[r].j;
        ids[r] = (float)j;
        probs[r] = sig[j] / (sum + FLT_EPSILON) * scaling;
    }
    for (int r = nsel; r < topk; ++r) { ids[r] = -1.0f; probs[r] = 0.0f; }
    return 0;
}

/* cpu.rs:528-572 */
int fo_moe_route(const float* logits, const float* bias, int n, int e, int topk, float routed_scaling,
                 float* probs, float* ids) {
    return fo_moe_route_grouped_nan(logits, bias, n, e, topk, 1, 1, routed_scaling, 0, probs, ids);
}

/*
 * Group-limited selection.  NOT in the reference (its router has no groups); this is the
 * DeepSeek-V3 form stated on top of cpu.rs:528-572:
 *   choice[j] = sigmoid(logit[j]) + bias[j]
 *   group g = experts [g*E/n_group, (g+1)*E/n_group); group score = largest + second-largest choice
 *   (f32 add, largest first; a one-expert group scores its only choice)
 *   keep the topk_group groups by (score desc, group index asc); experts outside them are excluded;
 *   then the reference's top-k / renormalisation over the kept experts.
 * n_group == 1 or topk_group == n_group keeps every expert and is exactly fo_moe_route.
 */
int fo_moe_route_grouped(const float* logits, const float* bias, int n, int e, int topk, int n_group,
                         int topk_group, float routed_scaling, float* probs, float* ids) {
    return fo_moe_route_grouped_nan(logits, bias, n, e, topk, n_group, topk_group, routed_scaling, 0, probs, ids);
}

/* The same with the NaN policy of route_row as a parameter.  Under policy 1 a NaN score takes no part in its
 * group's top-2 either (the comparisons that find them are false for NaN); a group without a finite score
 * scores -inf (-inf + -inf for two or more experts) and ranks after every group that has one. */
int fo_moe_route_grouped_nan(const float* logits, const float* bias, int n, int e, int topk, int n_group,
                             int topk_group, float routed_scaling, int nan_policy, float* probs, float* ids) {
    if (n < 0 || e <= 0 || topk <= 0 || topk > e) return 1;
    if (n_group > 1 && (e % n_group != 0 || topk_group <= 0 || topk_group > n_group)) return 1;
    int gs = n_group > 1 ? e / n_group : e;
    if (n_group > 1 && topk > topk_group * gs) return 1;
    float* sig = (float*)malloc(sizeof(float) * e);
    scored_t* sc = (scored_t*)malloc(sizeof(scored_t) * e);
    scored_t* gsc = (scored_t*)malloc(sizeof(scored_t) * (n_group > 1 ? n_group : 1));
    uint8_t* keep = (uint8_t*)malloc((size_t)e);
    int rc = 0;
    for (int i = 0; i < n && rc == 0; ++i) {
        const float* ls = logits + (size_t)i * e;
        if (n_group <= 1) {
            rc = route_row(ls, bias, e, topk, routed_scaling, NULL, nan_policy, sig, sc, probs + (size_t)i * topk,
                           ids + (size_t)i * topk);
            continue;
        }
        for (int g = 0; g < n_group; ++g) {
            float m1 = -INFINITY, m2 = -INFINITY;
            for (int j = g * gs; j < (g + 1) * gs; ++j) {
                float c = 1.0f / (1.0f + expf(-ls[j])) + bias[j];
                if (isnan(c) && nan_policy == 0) rc = 2;
                if (c > m1) { m2 = m1; m1 = c; }
                else if (c > m2) m2 = c;
            }
            gsc[g].s = gs > 1 ? m1 + m2 : m1;
            gsc[g].j = g;
        }
        if (rc) break;
        qsort(gsc, (size_t)n_group, sizeof(scored_t), scored_cmp);
        memset(keep, 0, (size_t)e);
        for (int r = 0; r < topk_group; ++r)
            for (int j = gsc[r].j * gs; j < (gsc[r].j + 1) * gs; ++j) keep[j] = 1;
        rc = route_row(ls, bias, e, topk, routed_scaling, keep, nan_policy, sig, sc, probs + (size_t)i * topk,
                       ids + (size_t)i * topk);
    }
    free(sig); free(sc); free(gsc); free(keep);
    return rc;
}

/* cpu.rs:574-625 (the iterator .sum::<f32>() folds from 0.0 in index order: the same chain) */
int fo_expert_ffn(const float* x, const float* gate_w, const float* up_w, const float* down_w, float limit,
                  float* out, int m, int hidden, int inter) {
    if (m < 0 || hidden <= 0 || inter <= 0) return 1;
    float* gu = (float*)malloc(sizeof(float) * 2 * (size_t)inter);
    float* act = (float*)malloc(sizeof(float) * (size_t)inter);
    for (int i = 0; i < m; ++i) {
        gemv_seq(x + (size_t)i * hidden, gate_w, hidden, inter, gu);
        gemv_seq(x + (size_t)i * hidden, up_w, hidden, inter, gu + inter);
        fo_swiglu_limited(gu, limit, act, 1, inter);
        gemv_seq(act, down_w, inter, hidden, out + (size_t)i * hidden);
    }
    free(gu); free(act);
    return 0;
}

/* ------------------------------------------------------------------ permutation */

/* kernels/cuda/dsv41_route.cu:194-225 (contract), :234-315 (construction): grouped order = expert
 * ascending, then flat assignment index i = t*topk + j ascending. */
int fo_moe_permute(const int32_t* ids, int n, int topk, int n_experts, int32_t* counts, int32_t* starts,
                   int32_t* perm_map, int32_t* gather_src, int32_t* active, int32_t* n_active) {
    if (n < 0 || topk <= 0 || n_experts <= 0) return 1;
    int n_assign = n * topk;
    int32_t* cursor = (int32_t*)malloc(sizeof(int32_t) * (size_t)n_experts);
    for (int e = 0; e < n_experts; ++e) counts[e] = 0;
    for (int g = 0; g < n_assign; ++g) gather_src[g] = -1;
    for (int i = 0; i < n_assign; ++i) {
        int e = ids[i];
        if (e >= 0 && e < n_experts) counts[e] += 1;
    }
    int acc = 0;
    for (int e = 0; e < n_experts; ++e) { starts[e] = acc; cursor[e] = acc; acc += counts[e]; }
    starts[n_experts] = acc;
    int na = 0;
    for (int e = 0; e < n_experts; ++e)
        if (counts[e] > 0) { if (active) active[na] = e; ++na; }
    if (active) for (int e = na; e < n_experts; ++e) active[e] = -1;
    if (n_active) *n_active = na;
    for (int i = 0; i < n_assign; ++i) {
        int e = ids[i];
        if (e < 0 || e >= n_experts) { perm_map[i] = -1; continue; }
        int g = cursor[e]++;
        perm_map[i] = g;
        gather_src[g] = i;
    }
    free(cursor);
    return 0;
}

/* crates/ferrite-models/src/dsv41/chain_dev.rs:862-899 */
int fo_moe_align_host(const int32_t* idx, int len, int topk, int seg_cap, int bm, int32_t* order,
                      int32_t* counts, int32_t* eid) {
    if (len <= 0 || topk == 0) return -1;
    for (int i = 0; i < len; ++i) if (idx[i] < 0) return -1;
    for (int i = 0; i < seg_cap * bm; ++i) order[i] = -1;
    for (int i = 0; i < seg_cap; ++i) { counts[i] = 0; eid[i] = 0; }
    /* stable sort of the index vector by expert: insertion sort keeps equal keys in flat order */
    int* perm = (int*)malloc(sizeof(int) * (size_t)len);
    for (int i = 0; i < len; ++i) {
        int j = i;
        while (j > 0 && idx[perm[j - 1]] > idx[i]) { perm[j] = perm[j - 1]; --j; }
        perm[j] = i;
    }
    int nseg = 0, a = 0;
    while (a < len) {
        if (nseg >= seg_cap) { free(perm); return -1; }
        int e = idx[perm[a]];
        int b = a;
        while (b < len && idx[perm[b]] == e) ++b;
        int run = b - a;
        if (run > bm) { free(perm); return -1; }
        for (int r = 0; r < run; ++r) order[nseg * bm + r] = perm[a + r];
        counts[nseg] = run;
        eid[nseg] = e;
        ++nseg;
        a = b;
    }
    free(perm);
    return nseg;
}

/* ------------------------------------------------------------------ the layer */

/* quantise-dequantise one row through act_quant_fp8(block 32, round_scale) (quant.rs:201-214) */
static void qdq_row_fp8(const float* x, int len, float* dst, uint8_t* tmpq, float* tmps) {
    fo_act_quant_fp8(x, (size_t)len, 32, 1, tmpq, tmps);
    for (int i = 0; i < len; ++i) dst[i] = fo_e4m3_decode(tmpq[i]) * tmps[i / 32];
}

/* Two-term form: q1/s1 = act_quant_fp8(x), q2/s2 = act_quant_fp8(x - decode(q1)*s1): x ~ dq1 + dq2.
 * The reference's e4m3 path quantises once (kernels.rs:97-108); the residual step is the one it uses for its e2m1
 * activations (out[i] = x[i] - decode(q[i]) * scale in f32, then the quantiser again: sub_dequant_fp4_kernel,
 * kernels/cuda/dsv41_kernels.cu:4165-4179), stated here with the e4m3 quantiser so that the device's two-term mode
 * has a bit-level definition. */
void fo_act_quant_fp8_x2(const float* x, size_t len, uint8_t* q1, float* s1, uint8_t* q2, float* s2) {
    float* r = (float*)malloc(sizeof(float) * len);
    fo_act_quant_fp8(x, len, 32, 1, q1, s1);
    for (size_t i = 0; i < len; ++i) r[i] = x[i] - fo_e4m3_decode(q1[i]) * s1[i / 32];
    fo_act_quant_fp8(r, len, 32, 1, q2, s2);
    free(r);
}

/* quantise-dequantise one row through the two-term quantiser: dst = dq1 + dq2 (one f32 addition) */
static void qdq_row_fp8_x2(const float* x, int len, float* dst) {
    uint8_t* q1 = (uint8_t*)malloc((size_t)len * 2);
    float* s1 = (float*)malloc(sizeof(float) * (size_t)(len / 32) * 2);
    uint8_t* q2 = q1 + len;
    float* s2 = s1 + len / 32;
    fo_act_quant_fp8_x2(x, (size_t)len, q1, s1, q2, s2);
    for (int i = 0; i < len; ++i)
        dst[i] = fo_e4m3_decode(q1[i]) * s1[i / 32] + fo_e4m3_decode(q2[i]) * s2[i / 32];
    free(q1); free(s1);
}

/* One expert applied to the rows listed in rows[] (token indices into xin).  y row r -> yout + r*H.
 * exec/lib.rs:1316-1332: gate = x.Wg^T, up = x.Wu^T, act = swiglu_limited([gate|up]), y = act.Wd^T. */
static void expert_rows(const fo_moe_cfg* cfg, const float* xin, const int* rows, int m, const float* wg,
                        const float* wu, const float* wd, int inter, float** ydst) {
    int H = cfg->hidden;
#pragma omp parallel num_threads(cfg->n_threads > 1 ? cfg->n_threads : 1)
    {
        float* gu = (float*)malloc(sizeof(float) * 2 * (size_t)inter);
        float* act = (float*)malloc(sizeof(float) * (size_t)inter);
        float* actq = (float*)malloc(sizeof(float) * (size_t)inter);
        uint8_t* tq = (uint8_t*)malloc((size_t)(inter > H ? inter : H));
        float* ts = (float*)malloc(sizeof(float) * (size_t)((inter > H ? inter : H) / 32 + 1));
#pragma omp for schedule(dynamic, 1)
        for (int r = 0; r < m; ++r) {
            const float* x = xin + (size_t)rows[r] * H;
            gemv_seq(x, wg, H, inter, gu);
            gemv_seq(x, wu, H, inter, gu + inter);
            fo_swiglu_limited(gu, cfg->swiglu_limit, act, 1, inter);
            const float* a = act;
            if (cfg->act_mode == 1) { qdq_row_fp8(act, inter, actq, tq, ts); a = actq; }
            else if (cfg->act_mode == 2) { qdq_row_fp8_x2(act, inter, actq); a = actq; }
            gemv_seq(a, wd, inter, H, ydst[r]);
        }
        free(gu); free(act); free(actq); free(tq); free(ts);
    }
}

int fo_moe_ffn_mxfp4(const fo_moe_cfg* cfg, const fo_moe_weights* w, const float* x, const int32_t* tok_sel,
                     int n_sel, float* out, float* logits_out, float* probs_out, float* ids_out) {
    const int n = cfg->n, H = cfg->hidden, E = cfg->n_experts, K = cfg->topk, I = cfg->inter, Is = cfg->shared_inter;
    if (n <= 0 || H % 32 || I % 32 || Is % 32 || K <= 0 || K > E) return 1;
    const int nt = cfg->n_threads > 1 ? cfg->n_threads : 1;
    int rc = 0;

    /* exec/lib.rs:1107 logits = x . gate.weight^T */
    float* logits = (float*)malloc(sizeof(float) * (size_t)n * E);
#pragma omp parallel for num_threads(nt) schedule(static)
    for (int t = 0; t < n; ++t) gemv_seq(x + (size_t)t * H, w->router_w, H, E, logits + (size_t)t * E);

    /* exec/lib.rs:1109-1116 bias (zeros when absent) + moe_route */
    float* bias = (float*)calloc((size_t)E, sizeof(float));
    if (w->router_bias) memcpy(bias, w->router_bias, sizeof(float) * (size_t)E);
    float* probs = (float*)malloc(sizeof(float) * (size_t)n * K);
    float* ids = (float*)malloc(sizeof(float) * (size_t)n * K);
    rc = fo_moe_route_grouped(logits, bias, n, E, K, cfg->n_group, cfg->topk_group, cfg->routed_scaling, probs, ids);
    if (logits_out) memcpy(logits_out, logits, sizeof(float) * (size_t)n * E);
    if (probs_out) memcpy(probs_out, probs, sizeof(float) * (size_t)n * K);
    if (ids_out) memcpy(ids_out, ids, sizeof(float) * (size_t)n * K);
    free(logits); free(bias);
    if (rc || !out) { free(probs); free(ids); return rc; }

    /* token subset */
    int ns = tok_sel ? n_sel : n;
    int* sel = (int*)malloc(sizeof(int) * (size_t)ns);
    for (int r = 0; r < ns; ++r) sel[r] = tok_sel ? tok_sel[r] : r;

    /* activations seen by the expert GEMMs */
    const float* xin = x;
    float* xq = NULL;
    if (cfg->act_mode == 1 || cfg->act_mode == 2) {
        xq = (float*)malloc(sizeof(float) * (size_t)n * H);
        uint8_t* tq = (uint8_t*)malloc((size_t)H);
        float* ts = (float*)malloc(sizeof(float) * (size_t)(H / 32));
        for (int r = 0; r < ns; ++r) {
            if (cfg->act_mode == 1) qdq_row_fp8(x + (size_t)sel[r] * H, H, xq + (size_t)sel[r] * H, tq, ts);
            else qdq_row_fp8_x2(x + (size_t)sel[r] * H, H, xq + (size_t)sel[r] * H);
        }
        free(tq); free(ts);
        xin = xq;
    }

    /* y[r][j][H]: expert output of selected token r, slot j.  The reference visits (j, eid) pairs and
     * adds probs*eout into out[t] (exec/lib.rs:1140-1161); for a fixed token that is one addition per
     * slot in ascending j starting from 0.0, which the combine below reproduces exactly. */
    float* y = (float*)malloc(sizeof(float) * (size_t)ns * K * H);
    float* wg = (float*)malloc(sizeof(float) * (size_t)(I > Is ? I : Is) * H);
    float* wu = (float*)malloc(sizeof(float) * (size_t)(I > Is ? I : Is) * H);
    float* wd = (float*)malloc(sizeof(float) * (size_t)(I > Is ? I : Is) * H);
    int* rows = (int*)malloc(sizeof(int) * (size_t)ns * K);
    float** ydst = (float**)malloc(sizeof(float*) * (size_t)ns * K);
    const size_t gsz = (size_t)I * (H / 2), gss = (size_t)I * (H / 32);
    const size_t dsz = (size_t)H * (I / 2), dss = (size_t)H * (I / 32);
    for (int e = 0; e < E; ++e) {
        int m = 0;
        for (int r = 0; r < ns; ++r)
            for (int j = 0; j < K; ++j)
                if ((int)ids[(size_t)sel[r] * K + j] == e) { rows[m] = sel[r]; ydst[m] = y + ((size_t)r * K + j) * H; ++m; }
        if (m == 0) continue;
        dequant_fp4_row32_mt(w->gate_w + e * gsz, w->gate_s + e * gss, (size_t)I, (size_t)H, wg, nt);
        dequant_fp4_row32_mt(w->up_w + e * gsz, w->up_s + e * gss, (size_t)I, (size_t)H, wu, nt);
        dequant_fp4_row32_mt(w->down_w + e * dsz, w->down_s + e * dss, (size_t)H, (size_t)I, wd, nt);
        expert_rows(cfg, xin, rows, m, wg, wu, wd, I, ydst);
    }

    /* shared expert over the selected tokens (exec/lib.rs:1130-1134) */
    float* shared = NULL;
    if (Is > 0) {
        shared = (float*)malloc(sizeof(float) * (size_t)ns * H);
        dequant_fp4_row32_mt(w->sh_gate_w, w->sh_gate_s, (size_t)Is, (size_t)H, wg, nt);
        dequant_fp4_row32_mt(w->sh_up_w, w->sh_up_s, (size_t)Is, (size_t)H, wu, nt);
        dequant_fp4_row32_mt(w->sh_down_w, w->sh_down_s, (size_t)H, (size_t)Is, wd, nt);
        for (int r = 0; r < ns; ++r) { rows[r] = sel[r]; ydst[r] = shared + (size_t)r * H; }
        expert_rows(cfg, xin, rows, ns, wg, wu, wd, Is, ydst);
    }

    /* exec/lib.rs:1154-1164: out[t] += probs[t,j] * eout (j ascending), then out += shared */
#pragma omp parallel for num_threads(nt) schedule(static)
    for (int r = 0; r < ns; ++r) {
        float* o = out + (size_t)r * H;
        for (int l = 0; l < H; ++l) o[l] = 0.0f;
        for (int j = 0; j < K; ++j) {
            float pw = probs[(size_t)sel[r] * K + j];
            const float* yr = y + ((size_t)r * K + j) * H;
            for (int l = 0; l < H; ++l) o[l] += pw * yr[l];
        }
        if (shared)
            for (int l = 0; l < H; ++l) o[l] += shared[(size_t)r * H + l];
    }
    free(y); free(wg); free(wu); free(wd); free(rows); free(ydst); free(shared); free(xq); free(sel);
    free(probs); free(ids);
    return 0;
}
