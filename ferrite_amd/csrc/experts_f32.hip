// f32 check mode of the expert FFN: activations stay f32, MXFP4 weights are dequantised exactly in
// registers, dot products accumulate in f32 FMA.  This path exists to compare the layer against the f32 CPU
// golden at 1e-5 (crates/ferrite-exec/src/lib.rs:1316-1332 for the expert, :1154-1164 for the combine); it
// re-reads an expert's weights once per routed row and is not the performance path.
//
// Rows are addressed in the grouped order of the permutation: row g < n*topk is assignment gather_src[g]
// (token = that / topk, expert = ids[that]); rows n*topk + t are the shared expert applied to token t.
#include "internal.hpp"
#include "numerics.hpp"

namespace fe {

// sum_l xs[l] * dequant(row)[l] over one MXFP4 row of K columns, whole wave cooperating; result in all lanes
__device__ __forceinline__ float mxfp4_row_dot(const uint8_t* __restrict__ codes, const uint8_t* __restrict__ scales,
                                               int K, const float* xs, int lane) {
    float acc = 0.0f;
    for (int off = lane * 4; off < K / 2; off += 256) {
        uint32_t v = *reinterpret_cast<const uint32_t*>(codes + off);
        int l = off * 2;
        float s = ue8m0_decode(scales[l >> 5]);
        const float4 x0 = *reinterpret_cast<const float4*>(xs + l);
        const float4 x1 = *reinterpret_cast<const float4*>(xs + l + 4);
        acc = fmaf(x0.x, e2m1_decode(v & 15u) * s, acc);
        acc = fmaf(x0.y, e2m1_decode((v >> 4) & 15u) * s, acc);
        acc = fmaf(x0.z, e2m1_decode((v >> 8) & 15u) * s, acc);
        acc = fmaf(x0.w, e2m1_decode((v >> 12) & 15u) * s, acc);
        acc = fmaf(x1.x, e2m1_decode((v >> 16) & 15u) * s, acc);
        acc = fmaf(x1.y, e2m1_decode((v >> 20) & 15u) * s, acc);
        acc = fmaf(x1.z, e2m1_decode((v >> 24) & 15u) * s, acc);
        acc = fmaf(x1.w, e2m1_decode((v >> 28) & 15u) * s, acc);
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) acc += __shfl_xor(acc, o, 64);
    return acc;
}

constexpr int F32_OUT_PER_BLOCK = 64;  // outputs per block (16 per wave)

struct RowSrc {
    int token;   // -1: empty row
    int expert;  // n_experts = shared
};

__device__ __forceinline__ RowSrc row_source(int g, int n, int topk, int n_experts, const int32_t* ids,
                                             const int32_t* gather_src) {
    RowSrc r;
    if (g >= n * topk) { r.token = g - n * topk; r.expert = n_experts; return r; }
    int i = gather_src[g];
    if (i < 0) { r.token = -1; r.expert = 0; return r; }
    r.token = i / topk;
    r.expert = ids[i];
    return r;
}

// act[g][i] = swiglu(x_t . Wg[e][i], x_t . Wu[e][i])
__global__ __launch_bounds__(256) void gate_up_f32_kernel(ferrite_moe_shape s, ferrite_moe_weights w,
                                                          const float* __restrict__ x, int n,
                                                          const int32_t* __restrict__ ids,
                                                          const int32_t* __restrict__ gather_src,
                                                          float* __restrict__ act) {
    extern __shared__ float xs[];
    const int g = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int H = s.hidden;
    RowSrc src = row_source(g, n, s.topk, s.n_experts, ids, gather_src);
    const bool shared = src.expert == s.n_experts;
    const int inter = shared ? s.shared_inter : s.inter;
    const int act_ld = s.inter > s.shared_inter ? s.inter : s.shared_inter;
    const int i0 = blockIdx.y * F32_OUT_PER_BLOCK;
    if (i0 >= inter) return;
    if (src.token < 0) {
        for (int i = threadIdx.x; i < F32_OUT_PER_BLOCK && i0 + i < inter; i += blockDim.x)
            act[(size_t)g * act_ld + i0 + i] = 0.0f;
        return;
    }
    for (int l = threadIdx.x; l < H; l += blockDim.x) xs[l] = x[(size_t)src.token * H + l];
    __syncthreads();
    const size_t mat_codes = (size_t)inter * (H / 2), mat_scales = (size_t)inter * (H / 32);
    const uint8_t* gw = shared ? w.sh_gate_w : w.gate_w + (size_t)src.expert * mat_codes;
    const uint8_t* gs = shared ? w.sh_gate_s : w.gate_s + (size_t)src.expert * mat_scales;
    const uint8_t* uw = shared ? w.sh_up_w : w.up_w + (size_t)src.expert * mat_codes;
    const uint8_t* us = shared ? w.sh_up_s : w.up_s + (size_t)src.expert * mat_scales;
    for (int r = wave; r < F32_OUT_PER_BLOCK; r += 4) {
        int i = i0 + r;
        if (i >= inter) break;
        float gv = mxfp4_row_dot(gw + (size_t)i * (H / 2), gs + (size_t)i * (H / 32), H, xs, lane);
        float uv = mxfp4_row_dot(uw + (size_t)i * (H / 2), us + (size_t)i * (H / 32), H, xs, lane);
        if (lane == 0) act[(size_t)g * act_ld + i] = swiglu_ref(gv, uv, s.swiglu_limit);
    }
}

// y[g][h] = act[g] . Wd[e][h]
__global__ __launch_bounds__(256) void down_f32_kernel(ferrite_moe_shape s, ferrite_moe_weights w,
                                                       const float* __restrict__ act, int n,
                                                       const int32_t* __restrict__ ids,
                                                       const int32_t* __restrict__ gather_src,
                                                       float* __restrict__ y) {
    extern __shared__ float xs[];
    const int g = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int H = s.hidden;
    RowSrc src = row_source(g, n, s.topk, s.n_experts, ids, gather_src);
    const bool shared = src.expert == s.n_experts;
    const int inter = shared ? s.shared_inter : s.inter;
    const int act_ld = s.inter > s.shared_inter ? s.inter : s.shared_inter;
    const int h0 = blockIdx.y * F32_OUT_PER_BLOCK;
    if (src.token < 0) {
        for (int i = threadIdx.x; i < F32_OUT_PER_BLOCK && h0 + i < H; i += blockDim.x) y[(size_t)g * H + h0 + i] = 0.0f;
        return;
    }
    for (int l = threadIdx.x; l < inter; l += blockDim.x) xs[l] = act[(size_t)g * act_ld + l];
    __syncthreads();
    const size_t mat_codes = (size_t)H * (inter / 2), mat_scales = (size_t)H * (inter / 32);
    const uint8_t* dw = shared ? w.sh_down_w : w.down_w + (size_t)src.expert * mat_codes;
    const uint8_t* ds = shared ? w.sh_down_s : w.down_s + (size_t)src.expert * mat_scales;
    for (int r = wave; r < F32_OUT_PER_BLOCK; r += 4) {
        int h = h0 + r;
        if (h >= H) break;
        float v = mxfp4_row_dot(dw + (size_t)h * (inter / 2), ds + (size_t)h * (inter / 32), inter, xs, lane);
        if (lane == 0) y[(size_t)g * H + h] = v;
    }
}

// out[t] = sum_j (ascending) probs[t,j] * y[perm_map[t*k+j]]  then  + y[n*k + t]   (exec/lib.rs:1154-1164:
// a rounded product and a rounded add per slot, the shared expert last)
// One 16-byte piece of a y row: four f32, or eight bf16 widened (exact).
template <typename YT>
struct YPiece {
    static constexpr int N = 16 / sizeof(YT);
    uint4 raw;
    __device__ __forceinline__ float at(int i) const {
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
        if constexpr (sizeof(YT) == 4) return u2f(w[i]);
        else return u2f((i & 1) ? (w[i >> 1] & 0xffff0000u) : (w[i >> 1] << 16));
    }
};

// f32 -> bf16, round to nearest even (NaN stays NaN)
__device__ __forceinline__ uint32_t combine_bf16(float f) {
    const uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

// A thread owns 16 bytes of every y row of its token (4 or 8 columns).  The slots are walked in batches of eight:
// first the eight table entries, then the eight row pieces - all loads of a batch are in flight together - then the
// products and sums in slot order.
// With hc.residual set (f32 output only) the token's combined row x is not stored: the hyper-connection update that
// follows the layer (KernelBackend::hc_post, cpu.rs:788-807) is applied to it in registers and its nh rows
// out[t,i,:] = post[t,i] * x + sum_k comb[t,k,i] * residual[t,k,:] (k ascending, multiply and add rounded
// separately) are what goes to memory.
template <typename OT, typename YT>
__global__ __launch_bounds__(256) void combine_kernel(const YT* __restrict__ y, const float* __restrict__ probs,
                                                      const int32_t* __restrict__ perm_map, int n, int topk,
                                                      int H, int has_shared, OT* __restrict__ out, HcPostArgs hc) {
    constexpr int N = YPiece<YT>::N;
    const int t = blockIdx.y;
    const int h = (blockIdx.x * blockDim.x + threadIdx.x) * N;
    if (h >= H) return;
    float o[N];
#pragma unroll
    for (int i = 0; i < N; ++i) o[i] = 0.0f;
    const int nk = n * topk;
    for (int j0 = 0; j0 < topk; j0 += 8) {
        int g[8];
        float p[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const bool in = j0 + j < topk;
            g[j] = in ? perm_map[(size_t)t * topk + j0 + j] : -1;
            p[j] = in ? probs[(size_t)t * topk + j0 + j] : 0.0f;
        }
        YPiece<YT> v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            // tables of an uninitialised workspace must not cause a fault: such slots are skipped
            const bool ok = g[j] >= 0 && g[j] < nk;
            v[j].raw = ok ? *reinterpret_cast<const uint4*>(y + (size_t)g[j] * H + h) : make_uint4(0u, 0u, 0u, 0u);
            g[j] = ok ? 1 : 0;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (g[j]) {
#pragma unroll
                for (int i = 0; i < N; ++i) o[i] = fadd(o[i], fmul(p[j], v[j].at(i)));
            }
        }
    }
    if (has_shared) {
        YPiece<YT> v;
        v.raw = *reinterpret_cast<const uint4*>(y + ((size_t)nk + t) * H + h);
#pragma unroll
        for (int i = 0; i < N; ++i) o[i] = fadd(o[i], v.at(i));
    }
    OT* dst = out + (size_t)t * H + h;
    if constexpr (sizeof(OT) == 4) {
        if (hc.residual != nullptr) {
            // the thread's columns of all nh residual streams first, as hc_post_kernel does: out may then be the
            // residual buffer itself (the in-place update of the streams)
            constexpr int MAX_NH = 8;
            const int nh = hc.nh;
            float rv[MAX_NH][N];
#pragma unroll
            for (int k = 0; k < MAX_NH; ++k) {
                if (k < nh) {
                    const float* r = hc.residual + ((size_t)t * nh + k) * H + h;
#pragma unroll
                    for (int c = 0; c < N; c += 4) {
                        const float4 q = *reinterpret_cast<const float4*>(r + c);
                        rv[k][c] = q.x; rv[k][c + 1] = q.y; rv[k][c + 2] = q.z; rv[k][c + 3] = q.w;
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < MAX_NH; ++i) {
                if (i >= nh) break;
                const float p = hc.post[(size_t)t * nh + i];
                float acc[N];
#pragma unroll
                for (int c = 0; c < N; ++c) acc[c] = fmul(p, o[c]);
#pragma unroll
                for (int k = 0; k < MAX_NH; ++k) {
                    if (k < nh) {
                        const float cf = hc.comb[((size_t)t * nh + k) * nh + i];
#pragma unroll
                        for (int c = 0; c < N; ++c) acc[c] = fadd(acc[c], fmul(cf, rv[k][c]));
                    }
                }
                float* od = reinterpret_cast<float*>(out) + ((size_t)t * nh + i) * H + h;
#pragma unroll
                for (int c = 0; c < N; c += 4)
                    *reinterpret_cast<float4*>(od + c) = make_float4(acc[c], acc[c + 1], acc[c + 2], acc[c + 3]);
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < N; i += 4) *reinterpret_cast<float4*>(dst + i) = make_float4(o[i], o[i + 1], o[i + 2], o[i + 3]);
    } else {
#pragma unroll
        for (int i = 0; i < N; i += 4)
            *reinterpret_cast<uint2*>(dst + i) = make_uint2(combine_bf16(o[i]) | (combine_bf16(o[i + 1]) << 16),
                                                            combine_bf16(o[i + 2]) | (combine_bf16(o[i + 3]) << 16));
    }
}

int launch_gate_up_f32(const ferrite_moe_shape& s, const ferrite_moe_weights& w, const float* x, int n,
                       const int32_t* ids, const int32_t* gather_src, float* act, hipStream_t st) {
    int rows = n * s.topk + (s.shared_inter > 0 ? n : 0);
    int imax = s.inter > s.shared_inter ? s.inter : s.shared_inter;
    dim3 grid(rows, (imax + F32_OUT_PER_BLOCK - 1) / F32_OUT_PER_BLOCK);
    gate_up_f32_kernel<<<grid, 256, (size_t)s.hidden * 4, st>>>(s, w, x, n, ids, gather_src, act);
    return check_launch("gate_up_f32");
}

int launch_down_f32(const ferrite_moe_shape& s, const ferrite_moe_weights& w, const float* act, int n,
                    const int32_t* ids, const int32_t* gather_src, float* y, hipStream_t st) {
    int rows = n * s.topk + (s.shared_inter > 0 ? n : 0);
    int imax = s.inter > s.shared_inter ? s.inter : s.shared_inter;
    dim3 grid(rows, (s.hidden + F32_OUT_PER_BLOCK - 1) / F32_OUT_PER_BLOCK);
    down_f32_kernel<<<grid, 256, (size_t)imax * 4, st>>>(s, w, act, n, ids, gather_src, y);
    return check_launch("down_f32");
}

int launch_combine(const void* y, int y_dtype, const float* probs, const int32_t* perm_map, int n, int topk,
                   int hidden, int has_shared, void* out, int out_dtype, hipStream_t st, const HcPostArgs* hcp) {
    const HcPostArgs hc = hcp ? *hcp : HcPostArgs{nullptr, nullptr, nullptr, 0};
    if (hc.residual && (out_dtype != FERRITE_DT_F32 || hc.nh < 1 || hc.nh > 8 || !hc.post || !hc.comb)) return FERRITE_ERR_INVALID_ARG;
    const bool of32 = out_dtype == FERRITE_DT_F32, yf32 = y_dtype == FERRITE_DT_F32;
    const int per_thread = yf32 ? 4 : 8;   // columns per thread: 16 bytes of a y row
    if (hidden % per_thread) return FERRITE_ERR_INVALID_ARG;
    dim3 grid((hidden / per_thread + 255) / 256, n);
    if ((!of32 && out_dtype != FERRITE_DT_BF16) || (!yf32 && y_dtype != FERRITE_DT_BF16)) return FERRITE_ERR_INVALID_ARG;
    if (of32 && yf32)
        combine_kernel<float, float><<<grid, 256, 0, st>>>((const float*)y, probs, perm_map, n, topk, hidden, has_shared, (float*)out, hc);
    else if (of32)
        combine_kernel<float, uint16_t><<<grid, 256, 0, st>>>((const uint16_t*)y, probs, perm_map, n, topk, hidden, has_shared, (float*)out, hc);
    else if (yf32)
        combine_kernel<uint16_t, float><<<grid, 256, 0, st>>>((const float*)y, probs, perm_map, n, topk, hidden, has_shared, (uint16_t*)out, hc);
    else
        combine_kernel<uint16_t, uint16_t><<<grid, 256, 0, st>>>((const uint16_t*)y, probs, perm_map, n, topk, hidden, has_shared, (uint16_t*)out, hc);
    return check_launch("combine");
}

}  // namespace fe
