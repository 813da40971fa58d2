// Router logits (bit-exact sequential-k f32 GEMM), noaux-tc sigmoid group-limited top-k, and the stable
// token permutation by expert.  gfx950, wave64.
#include "internal.hpp"
#include "device_utils.hpp"
#include "numerics.hpp"

namespace fe {

// ------------------------------------------------------------------------------------------------
// x . w^T with the reference's arithmetic (crates/ferrite-kernel/src/cpu.rs:106-111): for every output one
// chain s = 0; s = fl(s + fl(x[l] * w[l])) in ascending l.  The chain cannot be re-associated, so the
// kernel gives every output its own lane and only organises the operand traffic: a block owns 4 rows of x
// and 64 rows of w, stages 64-wide k-chunks of both through LDS (w transposed so that a lane reads four
// consecutive k of its own row with one 128-bit LDS read), and double-buffers the staging.
// ------------------------------------------------------------------------------------------------
constexpr int MM_TT = 4;    // x rows per block (one per wave)
constexpr int MM_TO = 64;   // w rows per block (one per lane)
constexpr int MM_KC = 64;   // k chunk
constexpr int MM_WPAD = MM_TO + 1;

__device__ __forceinline__ float load_x(const float* p, size_t i) { return p[i]; }
__device__ __forceinline__ float load_x(const uint16_t* p, size_t i) { return u2f((uint32_t)p[i] << 16); }

template <typename XT>
__global__ __launch_bounds__(256) void matmul_exact_kernel(const XT* __restrict__ x, const float* __restrict__ w,
                                                           const float* __restrict__ bias, float* __restrict__ out,
                                                           int n, int k, int o) {
    __shared__ float4 w_lds[2][MM_KC / 4][MM_WPAD];
    __shared__ float4 x_lds[2][MM_TT][MM_KC / 4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int o0 = blockIdx.x * MM_TO, t0 = blockIdx.y * MM_TT;
    const int nchunk = (k + MM_KC - 1) / MM_KC;

    // staging assignment: 64 w rows x 16 float4 per chunk = 1024 float4 -> 4 per thread; x: 4 x 16 = 64 float4
    float4 wreg[4];
    float4 xreg;
    auto fetch = [&](int c) {
        const int kb = c * MM_KC;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            int idx = tid + p * 256;
            int r = idx >> 4, c4 = idx & 15;
            int col = kb + c4 * 4;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (o0 + r < o) {
                const float* src = w + (size_t)(o0 + r) * k + col;
                if (col + 3 < k) v = *reinterpret_cast<const float4*>(src);
                else {
                    if (col < k) v.x = src[0];
                    if (col + 1 < k) v.y = src[1];
                    if (col + 2 < k) v.z = src[2];
                }
            }
            wreg[p] = v;
        }
        if (tid < MM_TT * (MM_KC / 4)) {
            int r = tid >> 4, c4 = tid & 15;
            int col = kb + c4 * 4;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (t0 + r < n) {
                size_t base = (size_t)(t0 + r) * k + col;
                if (col < k) v.x = load_x(x, base);
                if (col + 1 < k) v.y = load_x(x, base + 1);
                if (col + 2 < k) v.z = load_x(x, base + 2);
                if (col + 3 < k) v.w = load_x(x, base + 3);
            }
            xreg = v;
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            int idx = tid + p * 256;
            int r = idx >> 4, c4 = idx & 15;
            w_lds[buf][c4][r] = wreg[p];
        }
        if (tid < MM_TT * (MM_KC / 4)) x_lds[buf][tid >> 4][tid & 15] = xreg;
    };

    float s = 0.0f;
    fetch(0);
    stash(0);
    __syncthreads();
    for (int c = 0; c < nchunk; ++c) {
        const int buf = c & 1;
        if (c + 1 < nchunk) fetch(c + 1);
        const int klen = min(MM_KC, k - c * MM_KC);
        const int full4 = klen >> 2;
        for (int c4 = 0; c4 < full4; ++c4) {
            float4 wv = w_lds[buf][c4][lane];
            float4 xv = x_lds[buf][wave][c4];
            s = fadd(s, fmul(xv.x, wv.x));
            s = fadd(s, fmul(xv.y, wv.y));
            s = fadd(s, fmul(xv.z, wv.z));
            s = fadd(s, fmul(xv.w, wv.w));
        }
        if (klen & 3) {
            float4 wv = w_lds[buf][full4][lane];
            float4 xv = x_lds[buf][wave][full4];
            int rem = klen & 3;
            s = fadd(s, fmul(xv.x, wv.x));
            if (rem > 1) s = fadd(s, fmul(xv.y, wv.y));
            if (rem > 2) s = fadd(s, fmul(xv.z, wv.z));
        }
        if (c + 1 < nchunk) stash(buf ^ 1);
        __syncthreads();
    }
    const int t = t0 + wave, j = o0 + lane;
    if (t < n && j < o) {
        if (bias) s = fadd(s, bias[j]);
        out[(size_t)t * o + j] = s;
    }
}

int launch_matmul_exact(const void* x, int x_dtype, const float* w, const float* bias, float* out, int n, int k,
                        int o, hipStream_t st) {
    if (n < 0 || k < 0 || o < 0) return FERRITE_ERR_INVALID_ARG;
    if (n == 0 || o == 0) return FERRITE_OK;
    dim3 grid((o + MM_TO - 1) / MM_TO, (n + MM_TT - 1) / MM_TT);
    // the staging reads w with 128-bit loads: row starts must be 16-byte aligned
    if ((k & 3) != 0 || (reinterpret_cast<uintptr_t>(w) & 15) != 0) return FERRITE_DECLINED;
    if (x_dtype == FERRITE_DT_F32)
        matmul_exact_kernel<float><<<grid, 256, 0, st>>>((const float*)x, w, bias, out, n, k, o);
    else if (x_dtype == FERRITE_DT_BF16)
        matmul_exact_kernel<uint16_t><<<grid, 256, 0, st>>>((const uint16_t*)x, w, bias, out, n, k, o);
    else
        return FERRITE_ERR_INVALID_ARG;
    return check_launch("matmul_exact");
}

// Any-k variant: one lane per output straight from global memory (small or unaligned problems).
__global__ void matmul_exact_simple_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                           const float* __restrict__ bias, float* __restrict__ out, int n, int k,
                                           int o) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)n * o) return;
    int t = (int)(idx / o), j = (int)(idx % o);
    float s = 0.0f;
    for (int l = 0; l < k; ++l) s = fadd(s, fmul(x[(size_t)t * k + l], w[(size_t)j * k + l]));
    if (bias) s = fadd(s, bias[j]);
    out[idx] = s;
}

// ------------------------------------------------------------------------------------------------
// clamped SwiGLU (cpu.rs:178-203)
// ------------------------------------------------------------------------------------------------
__global__ void swiglu_kernel(const float* __restrict__ gate_up, float limit, float* __restrict__ out, int n,
                              int inter) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)n * inter) return;
    size_t i = idx / inter, j = idx % inter;
    out[idx] = swiglu_ref(gate_up[i * 2 * inter + j], gate_up[i * 2 * inter + inter + j], limit);
}

// ------------------------------------------------------------------------------------------------
// Routing: one wave per token.  sigmoid -> +bias -> (group top-2 sums -> keep topk_group groups) -> rank of
// every candidate under (choice desc, index asc) by counting the candidates that beat it -> the topk lowest
// ranks are the selection, in order -> renormalised weights from the raw sigmoid.
// Semantics and operation order follow cpu.rs:546-569; ties -> lower index (cpu.rs:560).
// ------------------------------------------------------------------------------------------------
constexpr int RT_MAX_E = 512;
constexpr int RT_MAX_K = 32;

__device__ __forceinline__ uint32_t ordered_u32(float f) {
    uint32_t u = f2u(f);
    return u ^ ((u >> 31) ? 0xFFFFFFFFu : 0x80000000u);
}

// LDS scratch of one routing wave
struct RouteScratch {
    unsigned long long key[RT_MAX_E];
    float choice[RT_MAX_E];
    float sel_sig[RT_MAX_K];
    int sel_id[RT_MAX_K];
    uint8_t keep[64];
};

// Loads that must observe stores made by other workgroups of the same kernel.
__device__ __forceinline__ float load_coherent(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ int load_coherent(const int32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Orders a wave's own LDS traffic: its lanes' earlier writes are visible to its later reads.  The LDS unit
// executes one wave's instructions in order, so only the compiler has to be kept from reordering.
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// One wave routes one token.  `lg` = the token's e logits.  The scratch is private to the wave, so waves of
// a block may call this independently of each other.
// NI = expert slots per lane (ceil(e / 64) rounded up to 1, 2, 4 or 8): everything below costs in proportion to it.
template <bool kCoherent, int NI>
__device__ __forceinline__ void route_wave_ni(const float* __restrict__ lg, const float* __restrict__ bias, bool live,
                                           int e, int topk, int n_group, int topk_group, float scaling,
                                           RouteScratch& sc, float* __restrict__ probs, float* __restrict__ ids_f32,
                                           int32_t* __restrict__ ids_i32) {
    const int lane = threadIdx.x & 63;
    const int ni = (e + 63) >> 6;
    float sg[NI], ch[NI];
    bool ok[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        int j = lane + 64 * i;
        ok[i] = live && i < ni && j < e;
        float l = 0.0f;
        if (ok[i]) l = kCoherent ? load_coherent(lg + j) : lg[j];
        sg[i] = sigmoid_ref(l);
        ch[i] = ok[i] ? fadd(sg[i], bias ? bias[j] : 0.0f) : 0.0f;
        // A NaN score (NaN logit or bias) is never selected, as in the reference's device router, whose arg-max
        // comparisons are false for NaN (kernels/cuda/ferrite_kernels.cu:1233-1241); slots that no finite score
        // can fill keep id -1 and weight 0 (ferrite_kernels.cu:1255-1270).  CpuBackend panics instead (cpu.rs:560).
        if (ch[i] != ch[i]) ok[i] = false;
    }
    if (lane < RT_MAX_K) { sc.sel_id[lane] = -1; sc.sel_sig[lane] = 0.0f; }

    if (n_group > 1) {
        const int gs = e / n_group;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            int j = lane + 64 * i;
            if (i < ni && j < e) sc.choice[j] = ch[i];
        }
        wave_sync();
        // lane g scores group g: largest + second largest choice (largest first)
        float gscore = 0.0f;
        if (lane < n_group) {
            float m1 = u2f(0xff800000u), m2 = u2f(0xff800000u);
            for (int j = lane * gs; j < (lane + 1) * gs; ++j) {
                float c = sc.choice[j];
                if (c > m1) { m2 = m1; m1 = c; }
                else if (c > m2) m2 = c;
            }
            gscore = gs > 1 ? fadd(m1, m2) : m1;
        }
        // rank of group g under (score desc, index asc)
        int rank = 0;
        for (int g2 = 0; g2 < n_group; ++g2) {
            float s2 = __shfl(gscore, g2, 64);
            rank += (s2 > gscore || (s2 == gscore && g2 < lane)) ? 1 : 0;
        }
        if (lane < n_group) sc.keep[lane] = rank < topk_group ? 1 : 0;
        wave_sync();
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            int j = lane + 64 * i;
            if (ok[i] && !sc.keep[j / gs]) ok[i] = false;
        }
    }

    // key = (order-preserving bits of choice, inverted index): larger key = earlier in the reference's sort
    unsigned long long key[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        uint32_t j = lane + 64 * i;
        key[i] = ok[i] ? (((unsigned long long)ordered_u32(ch[i]) << 32) | (0xFFFFFFFFu - j)) : 0ull;
        if (i < ni && (int)j < e) sc.key[j] = key[i];
    }
    wave_sync();
    int rank[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) rank[i] = 0;
    for (int j2 = 0; j2 < e; ++j2) {
        const unsigned long long kj = sc.key[j2];   // same address in every lane: an LDS broadcast
#pragma unroll
        for (int i = 0; i < NI; ++i) rank[i] += kj > key[i] ? 1 : 0;
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        if (key[i] != 0ull && rank[i] < topk) {
            sc.sel_id[rank[i]] = lane + 64 * i;
            sc.sel_sig[rank[i]] = sg[i];
        }
    }
    wave_sync();
    // cpu.rs:562-568: sum in selection order, then sig / (sum + f32::EPSILON) * scale
    float sum = 0.0f;
    for (int r = 0; r < topk; ++r) sum = fadd(sum, sc.sel_sig[r]);
    if (live && lane < topk) {
        const float my_sig = sc.sel_sig[lane];
        const int my_id = sc.sel_id[lane];
        probs[lane] = fmul(fdiv(my_sig, fadd(sum, 1.1920928955078125e-07f)), scaling);
        if (ids_f32) ids_f32[lane] = (float)my_id;
        if (ids_i32) ids_i32[lane] = my_id;
    }
}

template <bool kCoherent>
__device__ __forceinline__ void route_wave(const float* __restrict__ lg, const float* __restrict__ bias, bool live,
                                           int e, int topk, int n_group, int topk_group, float scaling,
                                           RouteScratch& sc, float* __restrict__ probs, float* __restrict__ ids_f32,
                                           int32_t* __restrict__ ids_i32) {
    if (e <= 64) route_wave_ni<kCoherent, 1>(lg, bias, live, e, topk, n_group, topk_group, scaling, sc, probs, ids_f32, ids_i32);
    else if (e <= 128) route_wave_ni<kCoherent, 2>(lg, bias, live, e, topk, n_group, topk_group, scaling, sc, probs, ids_f32, ids_i32);
    else if (e <= 256) route_wave_ni<kCoherent, 4>(lg, bias, live, e, topk, n_group, topk_group, scaling, sc, probs, ids_f32, ids_i32);
    else route_wave_ni<kCoherent, 8>(lg, bias, live, e, topk, n_group, topk_group, scaling, sc, probs, ids_f32, ids_i32);
}

__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits,
                                                        const float* __restrict__ bias, int n, int e, int topk,
                                                        int n_group, int topk_group, float scaling,
                                                        float* __restrict__ probs, float* __restrict__ ids_f32,
                                                        int32_t* __restrict__ ids_i32) {
    __shared__ RouteScratch scratch[4];
    const int wave = threadIdx.x >> 6;
    const int t = blockIdx.x * 4 + wave;
    const bool live = t < n;
    const size_t tt = live ? t : 0;
    route_wave<false>(logits + tt * e, bias, live, e, topk, n_group, topk_group, scaling, scratch[wave],
                      probs + tt * topk, ids_f32 ? ids_f32 + tt * topk : nullptr,
                      ids_i32 ? ids_i32 + tt * topk : nullptr);
}

// ------------------------------------------------------------------------------------------------
// Stable permutation by expert.  Every token holds each expert at most once, so the assignments of expert e
// in ascending flat index are its tokens in ascending order: rank = number of earlier tokens that chose e.
// Tokens are cut into chunks of 64; per (expert, chunk) a 64-bit membership mask is built with LDS atomics;
// a per-expert prefix over chunks plus a popcount below the token's bit gives the rank, and an exclusive
// scan of the per-expert totals gives the expert's first grouped row.  No global atomics and no dependence
// on scheduling: the tables are a pure function of ids.
//   phase A: masks    phase B: per-expert chunk prefixes, expert scan, active list, unit tables
//   phase C: scatter
// Small n runs A,B,C in one block with the masks in LDS; larger n uses three launches with the masks in the
// caller's scratch.
// ------------------------------------------------------------------------------------------------
constexpr int PM_MAX_E = 512;
constexpr int PM_SMALL_N = 1024;

struct PermArgs {
    const int32_t* ids;
    int n, topk, n_experts;
    int32_t *counts, *starts, *perm_map, *gather_src, *active, *n_active;
    int32_t *unit_expert, *unit_row0, *unit_rows, *unit_first, *unit_count, *n_units;
    int unit_cap, max_units, has_shared;
};

// How an expert's c rows are cut into `units` = ceil(c / cap) units.  With 16-row units the cut is every cap rows.
// The tiled kernels' units are balanced in whole 16-row tiles instead (the first `rem` units hold one tile more than
// the others): the blocks that work on the units of one expert then run at the same pace and fetch the expert's
// weights together, where a nearly empty last unit runs ahead of the full ones and both miss L2.
struct UnitCut {
    int c, cap, base, rem;   // base, rem: tiles per unit and units with one more (tiled kernels only)
    __device__ __forceinline__ UnitCut(int c_, int cap_, int units) : c(c_), cap(cap_), base(0), rem(0) {
        if (cap > 16 && units > 0) {
            const int tiles = (c + 15) >> 4;
            base = tiles / units;
            rem = tiles - base * units;
        }
    }
    __device__ __forceinline__ void span(int i, int& r0, int& rows) const {
        if (cap <= 16) {
            r0 = i * cap;
            rows = min(cap, c - r0);
        } else {
            r0 = (i * base + min(i, rem)) * 16;
            rows = min(c, r0 + (base + (i < rem ? 1 : 0)) * 16) - r0;
        }
    }
};

// wave 0 of a block: exclusive scan over experts + active list + unit tables. cnt[] readable by the wave.
__device__ void perm_expert_scan(const PermArgs& a, const int32_t* cnt, int32_t* starts_lds) {
    const int lane = threadIdx.x & 63;
    const int E = a.n_experts;
    const int per = (E + 63) >> 6;            // experts per lane (<= 8)
    const int e0 = lane * per;
    int tot = 0, nact = 0, ntile = 0;
    for (int i = 0; i < per; ++i) {
        int e = e0 + i;
        if (e < E) {
            int c = cnt[e];
            tot += c;
            nact += c > 0;
            if (a.unit_cap > 0) ntile += (c + a.unit_cap - 1) / a.unit_cap;
        }
    }
    // inclusive wave scans
    int s_tot = tot, s_act = nact, s_tile = ntile;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        int v0 = __shfl_up(s_tot, off, 64), v1 = __shfl_up(s_act, off, 64), v2 = __shfl_up(s_tile, off, 64);
        if (lane >= off) { s_tot += v0; s_act += v1; s_tile += v2; }
    }
    int run = s_tot - tot, ract = s_act - nact, rtile = s_tile - ntile;
    const int total = __shfl(s_tot, 63, 64), total_act = __shfl(s_act, 63, 64), total_tile = __shfl(s_tile, 63, 64);
    for (int i = 0; i < per; ++i) {
        int e = e0 + i;
        if (e < E) {
            int c = cnt[e];
            a.counts[e] = c;
            a.starts[e] = run;
            starts_lds[e] = run;
            if (c > 0 && a.active) a.active[ract] = e;
            ract += c > 0;
            if (a.unit_cap > 0) {
                const int first = rtile, cnt_e = (c + a.unit_cap - 1) / a.unit_cap;
                const UnitCut cut(c, a.unit_cap, cnt_e);
                for (int i2 = 0; i2 < cnt_e; ++i2) {
                    if (rtile < a.max_units) {
                        int r0, rows;
                        cut.span(i2, r0, rows);
                        a.unit_expert[rtile] = e;
                        a.unit_row0[rtile] = run + r0;
                        a.unit_rows[rtile] = rows;
                        if (a.unit_first) { a.unit_first[rtile] = first; a.unit_count[rtile] = cnt_e; }
                    }
                    ++rtile;
                }
            }
            run += c;
        }
    }
    if (lane == 0) {
        a.starts[E] = total;
        starts_lds[E] = total;
        if (a.n_active) *a.n_active = total_act;
    }
    if (a.active)
        for (int i = total_act + lane; i < E; i += 64) a.active[i] = -1;
    if (a.unit_cap > 0) {
        // shared expert: all n tokens, rows [n*topk, n*topk + n) of the activation / output row space
        int sh_tiles = a.has_shared ? (a.n + a.unit_cap - 1) / a.unit_cap : 0;
        const UnitCut sh_cut(a.n, a.unit_cap, sh_tiles);
        for (int i = lane; i < sh_tiles; i += 64) {
            int u = total_tile + i;
            if (u < a.max_units) {
                int r0, rows;
                sh_cut.span(i, r0, rows);
                a.unit_expert[u] = E;
                a.unit_row0[u] = a.n * a.topk + r0;
                a.unit_rows[u] = rows;
                if (a.unit_first) { a.unit_first[u] = total_tile; a.unit_count[u] = sh_tiles; }
            }
        }
        if (lane == 0) *a.n_units = min(total_tile + sh_tiles, a.max_units);
    }
}

static inline size_t perm_block_lds_bytes(int n, int n_experts) {
    size_t nchunk = ((size_t)n + 63) / 64;
    return (size_t)n_experts * nchunk * 12 + (size_t)(2 * n_experts + 1) * 4;
}

// The whole permutation by one workgroup (any multiple of 64 threads) or, with kWaveScope, by a single wave
// of a larger workgroup.  lds: perm_block_lds_bytes.
template <bool kCoherent, bool kWaveScope>
__device__ void permute_in_block(const PermArgs& a, unsigned long long* lds) {
    const int E = a.n_experts, n = a.n, k = a.topk;
    const int nchunk = (n + 63) >> 6;
    unsigned long long* mask = lds;                                      // [E][nchunk]
    int32_t* offs = reinterpret_cast<int32_t*>(mask + (size_t)E * nchunk);  // [E][nchunk]
    int32_t* cnt = offs + (size_t)E * nchunk;                            // [E]
    int32_t* starts_lds = cnt + E;                                       // [E+1]
    const int tid = kWaveScope ? (threadIdx.x & 63) : threadIdx.x, nthr = kWaveScope ? 64 : blockDim.x;
    auto sync = [] { if constexpr (kWaveScope) wave_sync(); else __syncthreads(); };
    auto id_at = [&](int i) -> int { return kCoherent ? load_coherent(a.ids + i) : a.ids[i]; };
    for (int i = tid; i < E * nchunk; i += nthr) mask[i] = 0ull;
    sync();
    for (int i = tid; i < n * k; i += nthr) {
        int t = i / k;
        int e = id_at(i);
        if (e >= 0 && e < E) atomicOr(&mask[(size_t)e * nchunk + (t >> 6)], 1ull << (t & 63));
    }
    sync();
    for (int e = tid; e < E; e += nthr) {
        int run = 0;
        for (int c = 0; c < nchunk; ++c) {
            offs[(size_t)e * nchunk + c] = run;
            run += __popcll(mask[(size_t)e * nchunk + c]);
        }
        cnt[e] = run;
    }
    sync();
    if (tid < 64) perm_expert_scan(a, cnt, starts_lds);
    sync();
    const int total = starts_lds[E];
    for (int i = tid; i < n * k; i += nthr) {
        int t = i / k;
        int e = id_at(i);
        if (e < 0 || e >= E) { a.perm_map[i] = -1; continue; }
        unsigned long long m = mask[(size_t)e * nchunk + (t >> 6)];
        int g = starts_lds[e] + offs[(size_t)e * nchunk + (t >> 6)] + __popcll(m & ((1ull << (t & 63)) - 1ull));
        a.perm_map[i] = g;
        a.gather_src[g] = i;
    }
    for (int g = total + tid; g < n * k; g += nthr) a.gather_src[g] = -1;
}

__global__ __launch_bounds__(1024) void permute_small_kernel(PermArgs a) {
    extern __shared__ unsigned long long pm_lds[];
    permute_in_block<false, false>(a, pm_lds);
}

// large-n phase A: one wave per 64-token chunk
__global__ __launch_bounds__(256) void permute_mask_kernel(PermArgs a, unsigned long long* __restrict__ gmask) {
    extern __shared__ unsigned long long pm_lds[];
    const int E = a.n_experts, n = a.n, k = a.topk;
    const int nchunk = (n + 63) >> 6;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int chunk = blockIdx.x * 4 + wave;
    unsigned long long* m = pm_lds + (size_t)wave * E;
    for (int e = lane; e < E; e += 64) m[e] = 0ull;
    __syncthreads();
    int t = chunk * 64 + lane;
    if (chunk < nchunk && t < n)
        for (int j = 0; j < k; ++j) {
            int e = a.ids[(size_t)t * k + j];
            if (e >= 0 && e < E) atomicOr(&m[e], 1ull << lane);
        }
    __syncthreads();
    if (chunk < nchunk)
        for (int e = lane; e < E; e += 64) gmask[(size_t)e * nchunk + chunk] = m[e];
}

// large-n phase B: one block; thread e walks its chunks
__global__ __launch_bounds__(512) void permute_scan_kernel(PermArgs a, const unsigned long long* __restrict__ gmask,
                                                           int32_t* __restrict__ goffs) {
    __shared__ int32_t cnt[PM_MAX_E];
    __shared__ int32_t starts_lds[PM_MAX_E + 1];
    const int E = a.n_experts;
    const int nchunk = (a.n + 63) >> 6;
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        int run = 0;
        const unsigned long long* me = gmask + (size_t)e * nchunk;
        int32_t* oe = goffs + (size_t)e * nchunk;
        int c = 0;
        for (; c + 8 <= nchunk; c += 8) {   // eight loads in flight: the walk is memory latency
            unsigned long long m[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) m[j] = me[c + j];
#pragma unroll
            for (int j = 0; j < 8; ++j) { oe[c + j] = run; run += __popcll(m[j]); }
        }
        for (; c < nchunk; ++c) { oe[c] = run; run += __popcll(me[c]); }
        cnt[e] = run;
    }
    __syncthreads();
    if (threadIdx.x < 64) perm_expert_scan(a, cnt, starts_lds);
}

// large-n phase C
__global__ __launch_bounds__(256) void permute_scatter_kernel(PermArgs a, const unsigned long long* __restrict__ gmask,
                                                              const int32_t* __restrict__ goffs) {
    const int E = a.n_experts, n = a.n, k = a.topk;
    const int nchunk = (n + 63) >> 6;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)n * k) return;
    const int total = a.starts[E];
    if ((int)i >= total) a.gather_src[i] = -1;   // positions no assignment reaches (distinct from any g below)
    int t = (int)(i / k);
    int e = a.ids[i];
    if (e < 0 || e >= E) { a.perm_map[i] = -1; return; }
    unsigned long long m = gmask[(size_t)e * nchunk + (t >> 6)];
    int g = a.starts[e] + goffs[(size_t)e * nchunk + (t >> 6)] + __popcll(m & ((1ull << (t & 63)) - 1ull));
    a.perm_map[i] = g;
    a.gather_src[g] = (int)i;
}

// ------------------------------------------------------------------------------------------------
// The head of the layer as ONE launch (decode-sized batches), or the router GEMM alone (kFused = false).
// Workgroups have eight waves.
//   blocks (eb, tg), eb < eblocks: router logits of the tokens of group tg for experts [64 eb, 64 eb + 64): the reference's
//                                  sequential chain, one lane of wave 0 per expert.  A lone wave issues one
//                                  instruction every four cycles, loads and address arithmetic included, so the
//                                  chain wave is left with nothing but the adds: six producer waves fetch the router
//                                  weight (k-blocked transpose [H/4][Epad][4], four chunks ahead), multiply it
//                                  with x[t] (the products are order-independent and each rounded once, as in
//                                  the reference) and hand the products over through a two-buffer LDS ring;
//                                  wave 0 reads them back and adds them in k order.  When one token per
//                                  block would need more than one round of blocks, a block takes two tokens
//                                  (two interleaved chains in wave 0, the weights fetched once for both)
//   blocks (eblocks, t)          : e4m3-per-32 quantisation of x[t] (off the critical path)
//   last logits block of a token : its wave 0 routes the token (arrival counter per token)
//   last routed token            : its block builds the permutation and unit tables with all of its waves (the
//                                  others have been waiting at a barrier for the chain wave's verdict) and clears
//                                  the counters so the next launch (or graph replay) starts clean
// counters[0] = routed tokens, counters[1 + t] = logits blocks of token t that have arrived; all zero on entry.
// ------------------------------------------------------------------------------------------------
constexpr int HEAD_MAX_N = 256;
constexpr int HD_NP = 6;                               // producer waves

struct HeadArgs {
    const void* x;
    const float* wt;      // [H/4][Epad][4]
    const float* bias;
    int n, H, E, Epad, topk, n_group, topk_group;
    float scaling;
    float *logits, *probs, *ids_f32;
    int32_t* ids;
    ActPlanes xq;         // q may be NULL: no quantisation blocks are launched then; q2 set: two-term
    int32_t* counters;    // [1 + n]
    int fuse_perm;        // the block that routes the last token also builds the permutation; else a separate launch does
    const float* norm_w;  // not NULL: x is the un-normalised f32 stream and every block applies rmsnorm(x, norm_w, eps)
    float eps;            // to its token(s) first (cpu.rs:124-143), so the normalised activations never go through HBM
    PermArgs perm;
};

// T = tokens per block, W = product groups (of four k, all tokens together) per ring buffer.
//   up to 256 blocks (one per CU)  : T 1, W 32 - 64 KiB of ring, the fewest barriers per chain
//   up to 512 blocks               : T 1, W 16 - 32 KiB of ring and under 128 registers, so two blocks share a CU and
//                                    their chain waves run side by side (192 tokens x 2 expert blocks: 44.7 us
//                                    against 60.6 us for two interleaved chains per block)
//   more                           : T 2, W 32 - two interleaved chains per block, the weights fetched once
template <int T, int W>
struct HeadCfg {
    static constexpr int CH = W / T;                         // groups of four k per chunk and token
    static constexpr int PW = (CH + HD_NP - 1) / HD_NP;      // groups per producer wave and chunk
    static constexpr size_t RING_BYTES = 2 * (size_t)W * 1024;
};

template <int T, int W>
struct HeadSet {
    float4 w[HeadCfg<T, W>::PW];
};

// Producer P (0..HD_NP-1) owns groups P, P+HD_NP, ... of every chunk.  Chunks past the end re-read the last one
// (never consumed), which keeps every load unconditional.
template <int T, int W, int P>
__device__ __forceinline__ void head_pload(HeadSet<T, W>& st, const float4* __restrict__ wp, int Epad, int c, int nch) {
    constexpr int CH = HeadCfg<T, W>::CH;
    const float4* base = wp + (size_t)min(c, nch - 1) * CH * Epad;
#pragma unroll
    for (int i = 0; i < HeadCfg<T, W>::PW; ++i)
        if (P + HD_NP * i < CH) st.w[i] = base[(size_t)(P + HD_NP * i) * Epad];
}

// products of the chunk's group j for token ti go to slot (j*T + ti)*64 + lane of the ring buffer
template <int T, int W, int P>
__device__ __forceinline__ void head_pmul(const HeadSet<T, W>& st, const float4* xl, int nk4, int c, float4* buf, int lane) {
    constexpr int CH = HeadCfg<T, W>::CH;
#pragma unroll
    for (int i = 0; i < HeadCfg<T, W>::PW; ++i) {
        const int j = P + HD_NP * i;
        if (j < CH) {
            const float4 wv = st.w[i];
#pragma unroll
            for (int ti = 0; ti < T; ++ti) {
                const float4 xv = xl[ti * nk4 + c * CH + j];
                buf[(j * T + ti) * 64 + lane] =
                    make_float4(fmul(xv.x, wv.x), fmul(xv.y, wv.y), fmul(xv.z, wv.z), fmul(xv.w, wv.w));
            }
        }
    }
}

// rmsnorm of the block's token(s) in place of the first barrier ("x is in LDS") of every wave's role.  On entry
// every thread has staged its share of the raw rows in xl and of their squares (each rounded once) in sq.  The
// reference sums the squares of a row left to right in f32 (cpu.rs:124-143): a serial chain, walked by wave 0 with
// 16-byte broadcast reads in counted batches, while the producer waves' first weight loads are already in flight.
// Then all waves scale xl to (x * inv) * w, which is what the router chain and the quantisation see.
struct HeadNorm {
    const float* w;
    float eps;
    float4* xl;
    const float4* sq;
    float* inv;   // [T] in LDS
    int nk4, T;
};

__device__ __forceinline__ void head_first_sync(const HeadNorm& nm) {
    __syncthreads();   // x (and with a norm the squares) are in LDS
    if (nm.w == nullptr) return;
    const int tid = threadIdx.x;
    if (tid < 64) {
        for (int ti = 0; ti < nm.T; ++ti) {
            float ss = sumsq_walk(nm.sq + (size_t)ti * nm.nk4, nm.nk4, 0.0f);
            ss = fdiv(ss, (float)(nm.nk4 * 4));
            const float inv = fdiv(1.0f, fsqrt(fadd(ss, nm.eps)));
            if (tid == 0) nm.inv[ti] = inv;
        }
    }
    __syncthreads();
    for (int i = tid; i < nm.T * nm.nk4; i += blockDim.x) {
        const int ti = i / nm.nk4, k4 = i - ti * nm.nk4;
        const float iv = nm.inv[ti];
        const float4 v = nm.xl[i], g = reinterpret_cast<const float4*>(nm.w)[k4];
        nm.xl[i] = make_float4(fmul(fmul(v.x, iv), g.x), fmul(fmul(v.y, iv), g.y), fmul(fmul(v.z, iv), g.z),
                               fmul(fmul(v.w, iv), g.w));
    }
    __syncthreads();   // the normalised rows are in place and the squares' space is free for the products
}

// Products of chunk c+1 are made while the chain consumes chunk c; register set c%4 holds the weights of chunk c
// and is reloaded for chunk c+4 as soon as it has been used.
template <int T, int W, int P>
__device__ __forceinline__ void head_producer(const float4* __restrict__ wp, int Epad, int nk4, const float4* xl,
                                              float4* ring, int lane, const HeadNorm& nm) {
    constexpr int CH = HeadCfg<T, W>::CH;
    const int nch = nk4 / CH;
    float4* b0 = ring;
    float4* b1 = ring + CH * T * 64;
    HeadSet<T, W> s0, s1, s2, s3;
    head_pload<T, W, P>(s0, wp, Epad, 0, nch);
    head_pload<T, W, P>(s1, wp, Epad, 1, nch);
    head_pload<T, W, P>(s2, wp, Epad, 2, nch);
    head_pload<T, W, P>(s3, wp, Epad, 3, nch);
    head_first_sync(nm);   // x is in LDS
    head_pmul<T, W, P>(s0, xl, nk4, 0, b0, lane);
    head_pload<T, W, P>(s0, wp, Epad, 4, nch);
    __syncthreads();
    for (int c = 0; c < nch; c += 4) {
        head_pmul<T, W, P>(s1, xl, nk4, min(c + 1, nch - 1), b1, lane);
        head_pload<T, W, P>(s1, wp, Epad, c + 5, nch);
        __syncthreads();
        head_pmul<T, W, P>(s2, xl, nk4, min(c + 2, nch - 1), b0, lane);
        head_pload<T, W, P>(s2, wp, Epad, c + 6, nch);
        __syncthreads();
        head_pmul<T, W, P>(s3, xl, nk4, min(c + 3, nch - 1), b1, lane);
        head_pload<T, W, P>(s3, wp, Epad, c + 7, nch);
        __syncthreads();
        head_pmul<T, W, P>(s0, xl, nk4, min(c + 4, nch - 1), b0, lane);
        head_pload<T, W, P>(s0, wp, Epad, c + 8, nch);
        __syncthreads();
    }
}

// The chains over one chunk of products: batches of eight LDS reads (8/T groups of four k for each of the T
// tokens), one wait per batch (0xC87F: lgkmcnt <= 8, i.e. everything but the batch just issued; 0xC07F: lgkmcnt 0),
// 32 adds per batch, dependent within a token's chain.
template <int T, int W>
__device__ __forceinline__ void head_consume(float (&s)[T], const float4* buf, int lane) {
    constexpr int NB = HeadCfg<T, W>::CH * T / 8;   // batches per chunk (4)
    float4 r[2][8];
#pragma unroll
    for (int j = 0; j < 8; ++j) r[0][j] = buf[j * 64 + lane];
#pragma unroll
    for (int g = 0; g < NB; ++g) {
        if (g + 1 < NB) {
#pragma unroll
            for (int j = 0; j < 8; ++j) r[(g + 1) & 1][j] = buf[((g + 1) * 8 + j) * 64 + lane];
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0xC87F);
        } else {
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0xC07F);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {   // slot order is (group, token): j % T is the token
            const float4 p = r[g & 1][j];
            float a = s[j % T];
            a = fadd(a, p.x);
            a = fadd(a, p.y);
            a = fadd(a, p.z);
            a = fadd(a, p.w);
            s[j % T] = a;
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

// Barriers pair one to one with head_producer's.
template <int T, int W>
__device__ __forceinline__ void head_consumer(float (&s)[T], int nk4, const float4* ring, int lane, const HeadNorm& nm) {
    constexpr int CH = HeadCfg<T, W>::CH;
    const int nch = nk4 / CH;
    const float4* b0 = ring;
    const float4* b1 = ring + CH * T * 64;
    __builtin_amdgcn_s_setprio(3);   // ahead of another block's producer waves on the same SIMD
    head_first_sync(nm);
    __syncthreads();
    for (int c = 0; c < nch; c += 4) {
        head_consume<T, W>(s, b0, lane);
        __syncthreads();
        if (c + 1 < nch) head_consume<T, W>(s, b1, lane);
        __syncthreads();
        if (c + 2 < nch) head_consume<T, W>(s, b0, lane);
        __syncthreads();
        if (c + 3 < nch) head_consume<T, W>(s, b1, lane);
        __syncthreads();
    }
    __builtin_amdgcn_s_setprio(0);
}

// The barriers of head_producer / head_consumer and nothing else.
template <int T, int W>
__device__ __forceinline__ void head_bystander(int nk4, const HeadNorm& nm) {
    const int nch = nk4 / HeadCfg<T, W>::CH;
    head_first_sync(nm);
    __syncthreads();
    for (int c = 0; c < nch; c += 4) {
        __syncthreads();
        __syncthreads();
        __syncthreads();
        __syncthreads();
    }
}

template <typename XT, bool kFused, int T, int W>
__global__ __launch_bounds__(512) void moe_head_kernel(HeadArgs a) {
    extern __shared__ __align__(16) unsigned char head_lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int eb = blockIdx.x, t0 = blockIdx.y * T;
    const int eblocks = a.Epad >> 6;
    const int H = a.H;
    if (eb == eblocks) {
        for (int ti = 0; ti < T; ++ti) {
            const int t = t0 + ti;
            if (t >= a.n) break;
            const XT* xrow = static_cast<const XT*>(a.x) + (size_t)t * H;
            if constexpr (sizeof(XT) == 4) {
                if (a.norm_w) {
                    // normalise the row in LDS first (the same three steps as in the logits blocks), quantise from there
                    float4* row = reinterpret_cast<float4*>(head_lds + HeadCfg<T, W>::RING_BYTES);
                    float4* sq = reinterpret_cast<float4*>(head_lds);
                    float* inv = reinterpret_cast<float*>(head_lds + HeadCfg<T, W>::RING_BYTES + (size_t)T * H * 4);
                    __syncthreads();   // the previous token's quantisation has read its row
                    for (int i = tid; i < H / 4; i += 512) {
                        const float4 v = reinterpret_cast<const float4*>(xrow)[i];
                        row[i] = v;
                        sq[i] = make_float4(fmul(v.x, v.x), fmul(v.y, v.y), fmul(v.z, v.z), fmul(v.w, v.w));
                    }
                    head_first_sync(HeadNorm{a.norm_w, a.eps, row, sq, inv, H / 4, 1});
                    xrow = reinterpret_cast<const XT*>(row);
                }
            }
            for (int b = tid; b < H / 32; b += 512) {
                const size_t at = (size_t)t * scale_pitch(H) + scale_pos(b), qo = (size_t)t * H + b * 32;
                if (a.xq.q2) {
                    const uint32_t sb = quant_block32_x2(xrow + b * 32, a.xq.q + qo, a.xq.q2 + qo);
                    a.xq.s[at] = (uint8_t)(sb & 0xffu);
                    a.xq.s2[at] = (uint8_t)(sb >> 8);
                } else {
                    a.xq.s[at] = (uint8_t)quant_block32(xrow + b * 32, a.xq.q + qo);
                }
            }
        }
        return;
    }
    float4* ring = reinterpret_cast<float4*>(head_lds);
    float4* xl = reinterpret_cast<float4*>(head_lds + HeadCfg<T, W>::RING_BYTES);   // [T][H/4]
    const int nk4 = H / 4;   // a multiple of 32 (H % 128 == 0)
    const float4* wp = reinterpret_cast<const float4*>(a.wt) + (size_t)eb * 64 + lane;
    for (int i = tid; i < T * nk4; i += 512) {
        const int ti = i / nk4, k4 = i - ti * nk4;
        const XT* xrow = static_cast<const XT*>(a.x) + (size_t)min(t0 + ti, a.n - 1) * H;
        float4 v;
        if constexpr (sizeof(XT) == 4) {
            v = reinterpret_cast<const float4*>(xrow)[k4];
        } else {
            uint2 q = reinterpret_cast<const uint2*>(xrow)[k4];
            v = make_float4(u2f(q.x << 16), u2f(q.x & 0xffff0000u), u2f(q.y << 16), u2f(q.y & 0xffff0000u));
        }
        xl[i] = v;
        if constexpr (sizeof(XT) == 4) {
            if (a.norm_w) ring[i] = make_float4(fmul(v.x, v.x), fmul(v.y, v.y), fmul(v.z, v.z), fmul(v.w, v.w));
        }
    }
    const HeadNorm nm{sizeof(XT) == 4 ? a.norm_w : nullptr, a.eps, xl, ring,
                      reinterpret_cast<float*>(head_lds + HeadCfg<T, W>::RING_BYTES + (size_t)T * H * 4), nk4, T};
    // wave 0 chains; wave 4 would share its SIMD (and its VALU issue slots) and only keeps the barriers company; the
    // others produce
    float s[T];
#pragma unroll
    for (int ti = 0; ti < T; ++ti) s[ti] = 0.0f;
    switch (wave) {
        case 0: head_consumer<T, W>(s, nk4, ring, lane, nm); break;
        case 1: head_producer<T, W, 0>(wp, a.Epad, nk4, xl, ring, lane, nm); break;
        case 2: head_producer<T, W, 1>(wp, a.Epad, nk4, xl, ring, lane, nm); break;
        case 3: head_producer<T, W, 2>(wp, a.Epad, nk4, xl, ring, lane, nm); break;
        case 5: head_producer<T, W, 3>(wp, a.Epad, nk4, xl, ring, lane, nm); break;
        case 6: head_producer<T, W, 4>(wp, a.Epad, nk4, xl, ring, lane, nm); break;
        case 7: head_producer<T, W, 5>(wp, a.Epad, nk4, xl, ring, lane, nm); break;
        default: head_bystander<T, W>(nk4, nm); break;
    }
    // From here on wave 0 works alone (LDS is free for its scratch); with a fused permutation the other waves wait
    // at the barrier below and join in if this block turns out to be the one that routed the last token.
    const bool block_perm = kFused && a.fuse_perm;
    if (wave != 0 && !block_perm) return;
    __shared__ int perm_here;
    int do_perm = 0;
    if (wave == 0) {
        const int e = eb * 64 + lane;
#pragma unroll
        for (int ti = 0; ti < T; ++ti) {
            const int t = t0 + ti;
            if (t >= a.n) break;
            if (e < a.E) a.logits[(size_t)t * a.E + e] = s[ti];
            if constexpr (kFused) {
                // arrival: the stores above are made visible before the counter moves
                __threadfence();
                int last = 0;
                if (lane == 0) last = atomicAdd(&a.counters[1 + t], 1) == eblocks - 1;
                last = __shfl(last, 0, 64);
                if (!last) continue;
                __threadfence();
                wave_sync();
                RouteScratch& sc = *reinterpret_cast<RouteScratch*>(head_lds);
                route_wave<true>(a.logits + (size_t)t * a.E, a.bias, true, a.E, a.topk, a.n_group, a.topk_group,
                                 a.scaling, sc, a.probs + (size_t)t * a.topk, a.ids_f32 + (size_t)t * a.topk,
                                 a.ids + (size_t)t * a.topk);
                __threadfence();
                last = 0;
                if (lane == 0) last = atomicAdd(&a.counters[0], 1) == a.n - 1;
                last = __shfl(last, 0, 64);
                if (!last) continue;
                __threadfence();
                wave_sync();
                do_perm = 1;
                for (int i = lane; i < a.n + 1; i += 64) a.counters[i] = 0;
            }
        }
        if (lane == 0) perm_here = do_perm;
    }
    if (!block_perm) return;
    __syncthreads();
    if (perm_here) permute_in_block<true, false>(a.perm, reinterpret_cast<unsigned long long*>(head_lds));
}

// tokens per block: two when one per block would not fit the chip's 256 CUs in one round
// (tokens per block, ring width) for n tokens x eblocks blocks of 64 experts: see HeadCfg.
struct HeadShape { int T, W; };
static HeadShape head_shape(int n, int eblocks) {
    const long blocks = (long)n * eblocks;
    // (the quantisation blocks, one more per token, are short but take a block slot each while they run: 96 tokens
    // x 2 blocks run in one round beside theirs, 37 us; 128 x 2 did not, 58 us against 44 us with the narrow ring)
    if (blocks + n / 2 <= 256) return {1, 32};
    if (blocks <= 512) return {1, 16};
    return {2, 32};
}

static size_t head_lds_bytes(int n, int H, int E, bool fused) {
    const HeadShape hs = head_shape(n, (E + 63) / 64);
    size_t b = 2 * (size_t)hs.W * 1024 + (size_t)hs.T * H * 4 + 64;   // ring, x rows, the rows' 1/rms
    if (fused) {
        if (b < sizeof(RouteScratch)) b = sizeof(RouteScratch);
        size_t p = perm_block_lds_bytes(n, E);
        if (p > b) b = p;
    }
    return b;
}

// The fused rmsnorm keeps the squares of the block's rows where the product ring will be.  Every block of a token
// walks that token's sum-of-squares chain again, which pays while each block has a CU to itself (32 tokens, H 4096:
// the block call 4 us shorter than with rmsnorm as a launch of its own) and no longer when two blocks share one
// (192 tokens: 6 us longer): offered for the one-block-per-CU shape only.
bool head_norm_supported(int n, int H, int E) {
    if (!head_supported(n, H, E)) return false;
    const HeadShape hs = head_shape(n, (E + 63) / 64);
    return hs.T == 1 && hs.W == 32 && (size_t)hs.T * H * 4 <= 2 * (size_t)hs.W * 1024;
}

bool head_supported(int n, int H, int E) {
    return n <= HEAD_MAX_N && E <= RT_MAX_E && (H % 128) == 0 && head_lds_bytes(n, H, E, true) <= 160 * 1024 - 64;   // 64: the kernel's static LDS
}

template <typename XT, bool kFused, int T, int W>
static int launch_head_tt(const HeadArgs& a, int quant, size_t lds, hipStream_t st) {
    int rc = LdsLimit<&moe_head_kernel<XT, kFused, T, W>>::ensure(lds);
    if (rc) return rc;
    dim3 grid(a.Epad / 64 + quant, (a.n + T - 1) / T);
    moe_head_kernel<XT, kFused, T, W><<<grid, 512, lds, st>>>(a);
    return check_launch("moe_head");
}

template <typename XT, bool kFused>
static int launch_head_t(const HeadArgs& a, int quant, size_t lds, hipStream_t st) {
    const HeadShape hs = head_shape(a.n, a.Epad / 64);
    if (hs.T == 2) return launch_head_tt<XT, kFused, 2, 32>(a, quant, lds, st);
    if (hs.W == 16) return launch_head_tt<XT, kFused, 1, 16>(a, quant, lds, st);
    return launch_head_tt<XT, kFused, 1, 32>(a, quant, lds, st);
}

int launch_moe_head(const void* x, int x_dtype, const float* router_t, const float* bias, const ferrite_moe_shape& s,
                    int n, float* logits, float* probs, float* ids_f32, int32_t* ids, const ActPlanes& xq,
                    int32_t* counters, int32_t* counts, int32_t* starts, int32_t* perm_map, int32_t* gather_src,
                    int32_t* active, int32_t* n_active, const UnitTables* units, int fuse_perm, const float* norm_w,
                    float eps, hipStream_t st) {
    if (!head_supported(n, s.hidden, s.n_experts)) return FERRITE_DECLINED;
    if (norm_w && (x_dtype != FERRITE_DT_F32 || !head_norm_supported(n, s.hidden, s.n_experts))) return FERRITE_DECLINED;
    HeadArgs a{};
    a.x = x; a.wt = router_t; a.bias = bias;
    a.n = n; a.H = s.hidden; a.E = s.n_experts; a.Epad = (s.n_experts + 63) / 64 * 64; a.topk = s.topk;
    a.n_group = (s.n_group > 1 && s.topk_group < s.n_group) ? s.n_group : 1;
    a.topk_group = s.topk_group; a.scaling = s.routed_scaling;
    a.logits = logits; a.probs = probs; a.ids_f32 = ids_f32; a.ids = ids; a.xq = xq; a.counters = counters;
    a.fuse_perm = fuse_perm;
    a.norm_w = norm_w; a.eps = eps;
    PermArgs& p = a.perm;
    p.ids = ids; p.n = n; p.topk = s.topk; p.n_experts = s.n_experts;
    p.counts = counts; p.starts = starts; p.perm_map = perm_map; p.gather_src = gather_src;
    p.active = active; p.n_active = n_active; p.has_shared = s.shared_inter > 0;
    if (units) {
        p.unit_expert = units->unit_expert; p.unit_row0 = units->unit_row0; p.unit_rows = units->unit_rows;
        p.unit_first = units->unit_first; p.unit_count = units->unit_count;
        p.n_units = units->n_units; p.unit_cap = units->unit_rows_cap; p.max_units = units->max_units;
    }
    const size_t lds = head_lds_bytes(n, s.hidden, s.n_experts, true);
    if (x_dtype == FERRITE_DT_F32) return launch_head_t<float, true>(a, xq.q ? 1 : 0, lds, st);
    if (x_dtype == FERRITE_DT_BF16) return launch_head_t<uint16_t, true>(a, xq.q ? 1 : 0, lds, st);
    return FERRITE_ERR_INVALID_ARG;
}

// What every routing kernel here assumes of its parameters, for the stand-alone op and for the fused head alike:
// argument errors first (the reference returns Err for them, cpu.rs:539-545), then the limits of these kernels
// (LDS arrays of RT_MAX_E keys, RT_MAX_K selections, one lane per group) as FERRITE_DECLINED.
int check_routing_params(int e, int topk, int n_group, int topk_group) {
    if (e <= 0 || topk <= 0 || topk > e) return FERRITE_ERR_INVALID_ARG;
    if (n_group > 1) {
        if (e % n_group != 0 || topk_group < 1 || topk_group > n_group) return FERRITE_ERR_INVALID_ARG;
        if (topk > topk_group * (e / n_group)) return FERRITE_ERR_INVALID_ARG;
        if (n_group > 64) return FERRITE_DECLINED;
    }
    if (e > RT_MAX_E || topk > RT_MAX_K) return FERRITE_DECLINED;
    return FERRITE_OK;
}

template <typename XT, bool kFused>
static int warmup_head() {
    const size_t cap = kLdsCap - 64;   // 64: the kernel's static LDS
    int rc;
    if ((rc = LdsLimit<&moe_head_kernel<XT, kFused, 1, 32>>::ensure(cap))) return rc;
    if ((rc = LdsLimit<&moe_head_kernel<XT, kFused, 1, 16>>::ensure(cap))) return rc;
    return LdsLimit<&moe_head_kernel<XT, kFused, 2, 32>>::ensure(cap);
}

template <typename XT> __global__ __launch_bounds__(256) void router_lds_kernel(const XT*, const float4*, int, int, int, int, float*);

int warmup_route() {
    int rc;
    if ((rc = LdsLimit<&router_lds_kernel<float>>::ensure(70 * 1024))) return rc;
    if ((rc = LdsLimit<&router_lds_kernel<uint16_t>>::ensure(70 * 1024))) return rc;
    if ((rc = warmup_head<float, true>())) return rc;
    if ((rc = warmup_head<uint16_t, true>())) return rc;
    if ((rc = warmup_head<float, false>())) return rc;
    return warmup_head<uint16_t, false>();
}

// Router GEMM for many tokens: the same sequential chain (cpu.rs:82-122), register tiled.  A wave owns 64 experts
// (one per lane, weights from the k-blocked transpose: one coalesced float4 per lane and four k) x T tokens whose
// activations are wave-uniform and therefore come through scalar loads; every (token, expert) pair still sees
// acc = acc + x*w for k ascending with separately rounded multiply and add.  T independent chains per lane cover
// the VALU latency.  grid (Epad/64, ceil(n / (4*T))), 4 waves per block on the same experts.
// One macro step = KM groups of four k: 16 k for bf16 activations, 8 k for f32, i.e. 32 bytes per token and step.
template <typename XT>
struct RouterStep {
    static constexpr int KM = sizeof(XT) == 4 ? 2 : 4;
};

template <typename XT, int T, int TE>
struct RouterSet {
    uint4 x[T][2];                            // 32 bytes of each token as loaded; wave-uniform -> scalar registers
    float4 w[RouterStep<XT>::KM][TE];
};

// Loads only: the bf16 -> f32 shifts happen at the use, so nothing here waits for the data.
template <typename XT, int T, int TE>
__device__ __forceinline__ void router_load(RouterSet<XT, T, TE>& r, const XT* const (&xr)[T], const float4* wp,
                                            int Epad, int step) {
    constexpr int KM = RouterStep<XT>::KM;
#pragma unroll
    for (int i = 0; i < T; ++i) {
        const uint4* p = reinterpret_cast<const uint4*>(xr[i]) + (size_t)step * 2;
        r.x[i][0] = p[0];
        r.x[i][1] = p[1];
    }
#pragma unroll
    for (int q = 0; q < KM; ++q)
#pragma unroll
        for (int j = 0; j < TE; ++j) r.w[q][j] = wp[(size_t)(step * KM + q) * Epad + j * 64];
}

template <typename XT, int T, int TE>
__device__ __forceinline__ void router_chain(float (&acc)[TE][T], const RouterSet<XT, T, TE>& r) {
    constexpr int KM = RouterStep<XT>::KM;
#pragma unroll
    for (int q = 0; q < KM; ++q) {
#pragma unroll
        for (int i = 0; i < T; ++i) {
            float x0, x1, x2, x3;
            if constexpr (sizeof(XT) == 4) {
                const uint4 v = r.x[i][q];
                x0 = u2f(v.x); x1 = u2f(v.y); x2 = u2f(v.z); x3 = u2f(v.w);
            } else {
                const uint4 v = r.x[i][q >> 1];
                const uint32_t lo = (q & 1) ? v.z : v.x, hi = (q & 1) ? v.w : v.y;
                x0 = u2f(lo << 16); x1 = u2f(lo & 0xffff0000u); x2 = u2f(hi << 16); x3 = u2f(hi & 0xffff0000u);
            }
#pragma unroll
            for (int j = 0; j < TE; ++j) {
                float a = acc[j][i];
                a = fadd(a, fmul(x0, r.w[q][j].x));
                a = fadd(a, fmul(x1, r.w[q][j].y));
                a = fadd(a, fmul(x2, r.w[q][j].z));
                a = fadd(a, fmul(x3, r.w[q][j].w));
                acc[j][i] = a;
            }
        }
    }
}

// TE blocks of 64 experts (lane = expert within the block) x T tokens per wave.
template <typename XT, int T, int TE>
__global__ __launch_bounds__(256) void router_tile_kernel(const XT* __restrict__ x, const float4* __restrict__ wt,
                                                          int n, int H, int E, int Epad, float* __restrict__ logits) {
    constexpr int KM = RouterStep<XT>::KM;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int t0 = (blockIdx.y * 4 + wave) * T;
    if (t0 >= n) return;
    const int e0 = blockIdx.x * 64 * TE + lane;
    const float4* wp = wt + e0;
    const XT* xr[T];
#pragma unroll
    for (int i = 0; i < T; ++i) xr[i] = x + (size_t)min(t0 + i, n - 1) * H;
    float acc[TE][T];
#pragma unroll
    for (int j = 0; j < TE; ++j)
#pragma unroll
        for (int i = 0; i < T; ++i) acc[j][i] = 0.0f;
    const int nsteps = H / (4 * KM);   // even: H % 128 == 0
    RouterSet<XT, T, TE> sa, sb;
    router_load(sa, xr, wp, Epad, 0);
    // Two register sets alternate: the loads of one are issued before the chains over the other.  Scalar loads
    // return out of order, so any wait on them is a wait for all of them: the set about to be used is waited
    // for BEFORE the other set's loads are issued (0xC07F: lgkmcnt 0, vmcnt and expcnt untouched).
    for (int st = 0; st < nsteps; st += 2) {
        __builtin_amdgcn_s_waitcnt(0xC07F);
        router_load(sb, xr, wp, Epad, st + 1);
        __builtin_amdgcn_sched_barrier(0);
        router_chain(acc, sa);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0xC07F);
        router_load(sa, xr, wp, Epad, min(st + 2, nsteps - 1));
        __builtin_amdgcn_sched_barrier(0);
        router_chain(acc, sb);
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int j = 0; j < TE; ++j) {
        const int e = e0 + j * 64;
        if (e < E) {
#pragma unroll
            for (int i = 0; i < T; ++i)
                if (t0 + i < n) logits[(size_t)(t0 + i) * E + e] = acc[j][i];
        }
    }
}

// The same chain for batches of a few hundred tokens, where the kernel above leaves SIMDs idle (four tokens per
// wave: 160 waves at 320 tokens x 128 experts, 115 us) or, with one token per wave, pulls every wave's own copy of
// the router weights through the vector memory path (1 KiB per wave and four k: 79 us, bound by the 64 bytes per
// clock a CU's address unit handles).  Here the four waves of a block work on four tokens against the same 64
// experts and share the weights through LDS: a chunk of RL_KC k (all 64 experts) is fetched once per block into a
// two-slot ring, a chunk ahead of its use, each wave stages its own token's activations (as f32) beside it, and a
// lane reads its expert's float4 and the token's float4 (a broadcast) per four k.  One barrier per chunk.
typedef float rl_f4 __attribute__((ext_vector_type(4)));
constexpr int RL_KC = 128;                                   // k per chunk
constexpr int RL_W_SLOT = RL_KC / 4 * 64;                    // float4 of weights per slot (32 KiB)
constexpr int RL_X_SLOT = 4 * RL_KC / 4;                     // float4 of activations per slot: 4 tokens x RL_KC f32
constexpr size_t RL_LDS_BYTES = 2 * (size_t)(RL_W_SLOT + RL_X_SLOT) * 16;

// A thread's share of chunk c: weight rows wave + 4 i of the chunk for expert e0 + lane, and two activations of the
// wave's token.
template <typename XT>
__device__ __forceinline__ void rl_fetch(rl_f4 (&wr)[RL_KC / 16], float (&xv)[2], const rl_f4* __restrict__ wt,
                                         const XT* __restrict__ xrow, int Epad, int col, int wave, int lane, int c) {
    const rl_f4* src = wt + (size_t)(c * (RL_KC / 4) + wave) * Epad + col;
#pragma unroll
    for (int i = 0; i < RL_KC / 16; ++i) wr[i] = src[(size_t)(4 * i) * Epad];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const XT v = xrow[c * RL_KC + i * 64 + lane];
        if constexpr (sizeof(XT) == 4) xv[i] = v; else xv[i] = u2f((uint32_t)v << 16);
    }
}

__device__ __forceinline__ void rl_stash(rl_f4* slot, const rl_f4 (&wr)[RL_KC / 16], const float (&xv)[2], int wave,
                                         int lane) {
#pragma unroll
    for (int i = 0; i < RL_KC / 16; ++i) slot[(wave + 4 * i) * 64 + lane] = wr[i];
    float* xs = reinterpret_cast<float*>(slot + RL_W_SLOT) + wave * RL_KC;
    xs[lane] = xv[0];
    xs[64 + lane] = xv[1];
}

template <typename XT>
__global__ __launch_bounds__(256) void router_lds_kernel(const XT* __restrict__ x, const float4* __restrict__ wt,
                                                         int n, int H, int E, int Epad, float* __restrict__ logits) {
    extern __shared__ __align__(16) unsigned char rl_raw[];
    rl_f4* lds = reinterpret_cast<rl_f4*>(rl_raw);
    const rl_f4* wt4 = reinterpret_cast<const rl_f4*>(wt);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int t = blockIdx.y * 4 + wave;
    const int col = blockIdx.x * 64 + lane;
    const XT* xrow = x + (size_t)min(t, n - 1) * H;
    const int nchunk = H / RL_KC;
    // One register set: chunk c + 1 is in flight while chunk c is walked.  What bounds a block is LDS bandwidth:
    // four waves read 1 KiB of weights each per four k, eight cycles per k, and with the chains' own instructions
    // on top a block takes 46-48 us at H 4096 (31 us with the multiplies compiled out).  Measured and not kept: a
    // second register set, a chunk fetched two chunk times ahead (67 us); the next group's LDS reads issued before
    // the current group's chain (46 us); the activations taken with v_readlane from registers instead of broadcast
    // LDS reads (50 us).
    rl_f4 wr[RL_KC / 16];
    float xv[2];
    float acc = 0.0f;
    rl_fetch(wr, xv, wt4, xrow, Epad, col, wave, lane, 0);
    rl_stash(lds, wr, xv, wave, lane);
    rl_fetch(wr, xv, wt4, xrow, Epad, col, wave, lane, min(1, nchunk - 1));
    for (int c = 0; c < nchunk; ++c) {
        __syncthreads();   // slot c % 2 is complete; nobody reads slot (c + 1) % 2 any more
        // past the last chunk both lines repeat it into the slot nobody reads any more: no branch around loads
        rl_stash(lds + ((c + 1) & 1) * (RL_W_SLOT + RL_X_SLOT), wr, xv, wave, lane);
        __builtin_amdgcn_sched_barrier(0);
        rl_fetch(wr, xv, wt4, xrow, Epad, col, wave, lane, min(c + 2, nchunk - 1));
        __builtin_amdgcn_sched_barrier(0);
        const rl_f4* w = lds + (c & 1) * (RL_W_SLOT + RL_X_SLOT);
        const rl_f4* xs = w + RL_W_SLOT + wave * (RL_KC / 4);
#pragma unroll 8
        for (int q = 0; q < RL_KC / 4; ++q) {
            const rl_f4 wq = w[q * 64 + lane], xq = xs[q];
            acc = fadd(acc, fmul(xq[0], wq[0]));
            acc = fadd(acc, fmul(xq[1], wq[1]));
            acc = fadd(acc, fmul(xq[2], wq[2]));
            acc = fadd(acc, fmul(xq[3], wq[3]));
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    if (t < n && col < E) logits[(size_t)t * E + col] = acc;
}

template <typename XT, int T>
static int launch_router_tile_t(const XT* xp, const float4* wp, int n, int H, int E, int Epad, float* logits,
                                hipStream_t st) {
    dim3 grid(1, (n + 4 * T - 1) / (4 * T));
    // two expert blocks per wave halve the weight traffic, but only when enough waves remain to hide latency
    if (Epad % 128 == 0 && (long)(Epad / 128) * grid.y * 4 >= 4096) {
        grid.x = Epad / 128;
        router_tile_kernel<XT, T, 2><<<grid, 256, 0, st>>>(xp, wp, n, H, E, Epad, logits);
    } else {
        grid.x = Epad / 64;
        router_tile_kernel<XT, T, 1><<<grid, 256, 0, st>>>(xp, wp, n, H, E, Epad, logits);
    }
    return check_launch("router_tile");
}

// Four tokens per wave in registers for thousands of tokens, two for a thousand or two (more waves), and the
// LDS-sharing kernel below that.
template <typename XT>
static int launch_router_tile(const void* x, const float* router_t, int n, int H, int E, float* logits, hipStream_t st) {
    const int Epad = (E + 63) / 64 * 64;
    const XT* xp = static_cast<const XT*>(x);
    const float4* wp = reinterpret_cast<const float4*>(router_t);
    const long groups = Epad / 64;
    // measured at 128 experts, H 4096: 320 / 512 / 767 / 1024 tokens 48 / 49 / 61 / 63 us with the LDS-sharing kernel
    // (79 / 80 / 85 / 86 us with one token per wave of the register-tiled kernel, 115 us with four); 1536 / 2048
    // tokens 97 / 98 us with two tokens per wave (101 / 117 us LDS-sharing, 115 / 116 us with four)
    if (groups * n <= 2048) {
        int rc = LdsLimit<&router_lds_kernel<XT>>::ensure(RL_LDS_BYTES);
        if (rc) return rc;
        dim3 grid((unsigned)groups, (n + 3) / 4);
        router_lds_kernel<XT><<<grid, 256, RL_LDS_BYTES, st>>>(xp, wp, n, H, E, Epad, logits);
        return check_launch("router_lds");
    }
    if (groups * n <= 4096) return launch_router_tile_t<XT, 2>(xp, wp, n, H, E, Epad, logits, st);
    return launch_router_tile_t<XT, 4>(xp, wp, n, H, E, Epad, logits, st);
}

// Router GEMM alone from the transposed weight (any n): logits only.
int launch_router_chain(const void* x, int x_dtype, const float* router_t, int n, int H, int E, float* logits,
                        hipStream_t st) {
    if (H % 128 != 0 || n <= 0 || n > 65535) return FERRITE_DECLINED;
    if (n >= 64) {
        if (x_dtype == FERRITE_DT_F32) return launch_router_tile<float>(x, router_t, n, H, E, logits, st);
        if (x_dtype == FERRITE_DT_BF16) return launch_router_tile<uint16_t>(x, router_t, n, H, E, logits, st);
        return FERRITE_ERR_INVALID_ARG;
    }
    if (head_lds_bytes(n, H, E, false) > 160 * 1024 - 64) return FERRITE_DECLINED;   // 64: the kernel's static LDS
    HeadArgs a{};
    a.x = x; a.wt = router_t; a.n = n; a.H = H; a.E = E; a.Epad = (E + 63) / 64 * 64; a.logits = logits;
    const size_t lds = head_lds_bytes(n, H, E, false);
    if (x_dtype == FERRITE_DT_F32) return launch_head_t<float, false>(a, 0, lds, st);
    if (x_dtype == FERRITE_DT_BF16) return launch_head_t<uint16_t, false>(a, 0, lds, st);
    return FERRITE_ERR_INVALID_ARG;
}

// router weight [E][H] -> k-blocked transpose [H/4][Epad][4], zero padded
__global__ __launch_bounds__(256) void router_transpose_kernel(const float* __restrict__ w, int E, int Epad, int H,
                                                               float4* __restrict__ dst) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)(H / 4) * Epad) return;
    int e = (int)(idx % Epad);
    size_t k4 = idx / Epad;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (e < E) v = *reinterpret_cast<const float4*>(w + (size_t)e * H + k4 * 4);
    dst[idx] = v;
}

int launch_router_transpose(const float* w, int E, int H, float* dst, hipStream_t st) {
    const int Epad = (E + 63) / 64 * 64;
    size_t total = (size_t)(H / 4) * Epad;
    router_transpose_kernel<<<(unsigned)((total + 255) / 256), 256, 0, st>>>(w, E, Epad, H, reinterpret_cast<float4*>(dst));
    return check_launch("router_transpose");
}

__global__ void zero_i32_kernel(int32_t* p, int count) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) p[i] = 0;
}

int launch_zero_i32(int32_t* p, int count, hipStream_t st) {
    if (count <= 0) return FERRITE_OK;
    zero_i32_kernel<<<(count + 255) / 256, 256, 0, st>>>(p, count);
    return check_launch("zero_i32");
}

size_t perm_scratch_bytes(int n, int n_experts) {
    size_t nchunk = ((size_t)n + 63) / 64;
    return (size_t)n_experts * nchunk * (8 + 4) + 64;
}

int launch_permute(const int32_t* ids, int n, int topk, int n_experts, int32_t* counts, int32_t* starts,
                   int32_t* perm_map, int32_t* gather_src, int32_t* active, int32_t* n_active, void* scratch,
                   size_t scratch_bytes, const UnitTables* units, int has_shared, hipStream_t st) {
    if (n <= 0 || topk <= 0 || n_experts <= 0 || n_experts > PM_MAX_E) return FERRITE_ERR_INVALID_ARG;
    PermArgs a{};
    a.ids = ids; a.n = n; a.topk = topk; a.n_experts = n_experts;
    a.counts = counts; a.starts = starts; a.perm_map = perm_map; a.gather_src = gather_src;
    a.active = active; a.n_active = n_active; a.has_shared = has_shared;
    if (units) {
        a.unit_expert = units->unit_expert; a.unit_row0 = units->unit_row0; a.unit_rows = units->unit_rows;
        a.unit_first = units->unit_first; a.unit_count = units->unit_count;
        a.n_units = units->n_units; a.unit_cap = units->unit_rows_cap; a.max_units = units->max_units;
    }
    const int nchunk = (n + 63) / 64;
    const size_t lds = perm_block_lds_bytes(n, n_experts);
    if (n <= PM_SMALL_N && lds <= 60 * 1024) {
        permute_small_kernel<<<1, 1024, lds, st>>>(a);
        return check_launch("permute_small");
    }
    if (scratch == nullptr || scratch_bytes < perm_scratch_bytes(n, n_experts)) return FERRITE_ERR_WORKSPACE;
    unsigned long long* gmask = reinterpret_cast<unsigned long long*>(scratch);
    int32_t* goffs = reinterpret_cast<int32_t*>(gmask + (size_t)n_experts * nchunk);
    permute_mask_kernel<<<(nchunk + 3) / 4, 256, (size_t)4 * n_experts * 8, st>>>(a, gmask);
    int rc = check_launch("permute_mask");
    if (rc) return rc;
    permute_scan_kernel<<<1, 512, 0, st>>>(a, gmask, goffs);
    rc = check_launch("permute_scan");
    if (rc) return rc;
    size_t na = (size_t)n * topk;
    permute_scatter_kernel<<<(unsigned)((na + 255) / 256), 256, 0, st>>>(a, gmask, goffs);
    return check_launch("permute_scatter");
}

}  // namespace fe

using namespace fe;

extern "C" int ferrite_matmul_f32(const float* x, const float* w, const float* bias, float* out, int n, int k,
                                  int o, ferrite_stream_t stream) {
    if (n < 0 || k < 0 || o < 0) return FERRITE_ERR_INVALID_ARG;
    if (n == 0 || o == 0) return FERRITE_OK;
    if ((n > 0 && !x) || !w || !out) return FERRITE_ERR_INVALID_ARG;
    hipStream_t st = as_stream(stream);
    if ((k & 3) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0 && (size_t)n * o >= 1024)
        return launch_matmul_exact(x, FERRITE_DT_F32, w, bias, out, n, k, o, st);
    size_t total = (size_t)n * o;
    matmul_exact_simple_kernel<<<(unsigned)((total + 63) / 64), 64, 0, st>>>(x, w, bias, out, n, k, o);
    return check_launch("matmul_exact_simple");
}

extern "C" int ferrite_swiglu_limited_f32(const float* gate_up, float limit, float* out, int n, int inter,
                                          ferrite_stream_t stream) {
    if (n < 0 || inter < 0) return FERRITE_ERR_INVALID_ARG;
    size_t total = (size_t)n * inter;
    if (total == 0) return FERRITE_OK;
    if (!gate_up || !out) return FERRITE_ERR_INVALID_ARG;
    swiglu_kernel<<<(unsigned)((total + 255) / 256), 256, 0, as_stream(stream)>>>(gate_up, limit, out, n, inter);
    return check_launch("swiglu");
}

extern "C" int ferrite_moe_route(const float* logits, const float* bias, int n, int e, int topk, int n_group,
                                 int topk_group, float routed_scaling, float* probs, float* ids_f32,
                                 int32_t* ids_i32, ferrite_stream_t stream) {
    if (n < 0 || !logits || !probs) return FERRITE_ERR_INVALID_ARG;
    if (int rc = check_routing_params(e, topk, n_group, topk_group)) return rc;
    if (n_group < 1 || topk_group == n_group) n_group = 1;  // keeps every expert: the ungrouped router
    if (n == 0) return FERRITE_OK;
    moe_route_kernel<<<(n + 3) / 4, 256, 0, as_stream(stream)>>>(logits, bias, n, e, topk, n_group, topk_group,
                                                                 routed_scaling, probs, ids_f32, ids_i32);
    return check_launch("moe_route");
}

extern "C" size_t ferrite_moe_permute_scratch_bytes(int n, int topk, int n_experts) {
    if (n <= 0 || topk <= 0 || n_experts <= 0 || (long long)n * topk > 0x3fffffffLL) return 0;
    return perm_scratch_bytes(n * topk, n_experts);
}

extern "C" int ferrite_moe_permute(const int32_t* ids, int n, int topk, int n_experts, int32_t* counts,
                                   int32_t* starts, int32_t* perm_map, int32_t* gather_src, int32_t* active,
                                   int32_t* n_active, void* scratch, size_t scratch_bytes,
                                   ferrite_stream_t stream) {
    if (!ids || !counts || !starts || !perm_map || !gather_src) return FERRITE_ERR_INVALID_ARG;
    if (n <= 0 || topk <= 0 || (long long)n * topk > 0x3fffffffLL) return FERRITE_ERR_INVALID_ARG;
    // The kernels rank an assignment by the earlier *tokens* that chose its expert, which is right when a token
    // holds each expert at most once (what a router emits).  This stand-alone op promises nothing about its ids
    // (the reference's own vector, chain_dev.rs:25042, lists an expert twice in one token), so it runs them with
    // every assignment as a token of its own: flat index, tables and order are the same, duplicates rank by slot.
    return launch_permute(ids, n * topk, 1, n_experts, counts, starts, perm_map, gather_src, active, n_active, scratch,
                          scratch_bytes, nullptr, 0, as_stream(stream));
}
