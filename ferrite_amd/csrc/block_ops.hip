// The steps on either side of the MoE FFN inside a decoder layer (crates/ferrite-exec/src/lib.rs:487-492):
// rmsnorm(post_attention_layernorm) in front of it and the hyper-connection update hc_post behind it, each
// reproducing the reference's f32 evaluation order bit for bit, and the three of them as one call.
#include <hip/hip_runtime.h>

#include "internal.hpp"
#include "device_utils.hpp"
#include "numerics.hpp"

namespace fe {

constexpr int RN_CHUNK = 4096;   // floats of one row staged in LDS at a time (16 KiB)

// KernelBackend::rmsnorm (crates/ferrite-kernel/src/cpu.rs:124-143).  The reference sums the squares of a row left
// to right in f32, so the sum is a serial chain of `dim` adds.  One wave per row: the lanes square 64 elements at a
// time into LDS (order-independent, each rounded once), then every lane walks the chain over the staged chunk with
// 16-byte broadcast reads (all lanes read the same address and hold the same running sum).  Second pass:
// out = (x * inv) * w.
__global__ __launch_bounds__(64) void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w, float eps,
                                                     float* __restrict__ out, int dim) {
    __shared__ __align__(16) float sq[RN_CHUNK];
    const int lane = threadIdx.x;
    const float* row = x + (size_t)blockIdx.x * dim;
    const bool vec4 = (dim & 3) == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) |
                                           reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    float ss = 0.0f;
    for (int base = 0; base < dim; base += RN_CHUNK) {
        const int len = min(RN_CHUNK, dim - base);
        const int len4 = (len + 3) & ~3;
        if (vec4) {
            // all of the lane's loads of the chunk are issued before the first square is written (16 in flight)
            const float4* r4 = reinterpret_cast<const float4*>(row + base);
            float4 v[RN_CHUNK / 256];
#pragma unroll
            for (int q = 0; q < RN_CHUNK / 256; ++q) {
                const int j4 = q * 64 + lane;
                v[q] = j4 * 4 < len ? r4[j4] : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int q = 0; q < RN_CHUNK / 256; ++q) {
                const int j4 = q * 64 + lane;
                if (j4 * 4 < len4)
                    reinterpret_cast<float4*>(sq)[j4] =
                        make_float4(fmul(v[q].x, v[q].x), fmul(v[q].y, v[q].y), fmul(v[q].z, v[q].z), fmul(v[q].w, v[q].w));
            }
        } else {
#pragma unroll 8
            for (int j = lane; j < len4; j += 64) {
                const float v = j < len ? row[base + j] : 0.0f;   // padding squares are +0: adding them changes nothing
                sq[j] = fmul(v, v);
            }
        }
        __syncthreads();
        ss = sumsq_walk(reinterpret_cast<const float4*>(sq), len4 / 4, ss);
        __syncthreads();
    }
    ss = fdiv(ss, (float)dim);
    const float inv = fdiv(1.0f, fsqrt(fadd(ss, eps)));
    float* orow = out + (size_t)blockIdx.x * dim;
    if (vec4) {
#pragma unroll 4
        for (int j4 = lane; j4 < dim / 4; j4 += 64) {
            const float4 v = reinterpret_cast<const float4*>(row)[j4], g = reinterpret_cast<const float4*>(w)[j4];
            reinterpret_cast<float4*>(orow)[j4] = make_float4(fmul(fmul(v.x, inv), g.x), fmul(fmul(v.y, inv), g.y),
                                                              fmul(fmul(v.z, inv), g.z), fmul(fmul(v.w, inv), g.w));
        }
    } else {
#pragma unroll 8
        for (int j = lane; j < dim; j += 64) orow[j] = fmul(fmul(row[j], inv), w[j]);
    }
}

// The same with four waves per row, for rows of up to 8192 16-byte-aligned floats: every thread keeps its part of
// the row and of w in registers (one pass over memory instead of two, four times the loads in flight), wave 0 walks
// the chain over the whole row's squares, the others wait.  At 192 rows of 4096 this takes 14.8 us against 21.5 us for
// one wave per row and the earlier form of the chain walk; the walk itself (4096 dependent adds and their 1024
// reads) is about 10 us.
constexpr int RN_ROW_MAX = 8192;

template <int NV>
__global__ __launch_bounds__(256, NV == 8 ? 2 : 4) void rmsnorm_row_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                          float eps, float* __restrict__ out, int dim) {
    extern __shared__ __align__(16) float sq[];   // the row's squares, zero padded to whole pieces of 256 values, + 1/rms
    const int tid = threadIdx.x;
    const int n4 = dim >> 2, pad4 = ((dim + 255) & ~255) >> 2;
    const float4* r4 = reinterpret_cast<const float4*>(x + (size_t)blockIdx.x * dim);
    const float4* w4 = reinterpret_cast<const float4*>(w);
    float4 v[NV], g[NV];
#pragma unroll
    for (int q = 0; q < NV; ++q) {
        const int j4 = q * 256 + tid;
        v[q] = j4 < n4 ? r4[j4] : make_float4(0.f, 0.f, 0.f, 0.f);   // padding squares are +0: adding them changes nothing
    }
#pragma unroll
    for (int q = 0; q < NV; ++q) {
        const int j4 = q * 256 + tid;
        g[q] = j4 < n4 ? w4[j4] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int q = 0; q < NV; ++q) {
        const int j4 = q * 256 + tid;
        if (j4 < pad4)
            reinterpret_cast<float4*>(sq)[j4] =
                make_float4(fmul(v[q].x, v[q].x), fmul(v[q].y, v[q].y), fmul(v[q].z, v[q].z), fmul(v[q].w, v[q].w));
    }
    __syncthreads();
    if (tid < 64) {
        float ss = sumsq_walk(reinterpret_cast<const float4*>(sq), pad4, 0.0f);
        ss = fdiv(ss, (float)dim);
        const float inv = fdiv(1.0f, fsqrt(fadd(ss, eps)));
        if (tid == 0) sq[pad4 * 4] = inv;
    }
    __syncthreads();
    const float inv = sq[pad4 * 4];
    float4* o4 = reinterpret_cast<float4*>(out + (size_t)blockIdx.x * dim);
#pragma unroll
    for (int q = 0; q < NV; ++q) {
        const int j4 = q * 256 + tid;
        if (j4 < n4)
            o4[j4] = make_float4(fmul(fmul(v[q].x, inv), g[q].x), fmul(fmul(v[q].y, inv), g[q].y),
                                 fmul(fmul(v[q].z, inv), g[q].z), fmul(fmul(v[q].w, inv), g[q].w));
    }
}

// KernelBackend::hc_post (cpu.rs:788-807; the CUDA counterpart is hc_post_kernel, kernels/cuda/ferrite_kernels.cu:2679):
// out[t,i,:] = post[t,i] * x[t,:] + sum_k comb[t,k,i] * residual[t,k,:], accumulated in k order with separately
// rounded multiply and add.  One thread per (token, 4 columns); the nh residual vectors stay in registers.
constexpr int HC_MAX_NH = 8;

__global__ __launch_bounds__(256) void hc_post_kernel(const float* __restrict__ x, const float* __restrict__ residual,
                                                      const float* __restrict__ post, const float* __restrict__ comb,
                                                      float* __restrict__ out, int nh, int h) {
    const int t = blockIdx.y;
    const int j = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (j >= h) return;
    const float4 xv = *reinterpret_cast<const float4*>(x + (size_t)t * h + j);
    float4 r[HC_MAX_NH];
#pragma unroll
    for (int k = 0; k < HC_MAX_NH; ++k)
        if (k < nh) r[k] = *reinterpret_cast<const float4*>(residual + ((size_t)t * nh + k) * h + j);
#pragma unroll
    for (int i = 0; i < HC_MAX_NH; ++i) {
        if (i >= nh) break;
        const float p = post[(size_t)t * nh + i];
        float4 acc = make_float4(fmul(p, xv.x), fmul(p, xv.y), fmul(p, xv.z), fmul(p, xv.w));
#pragma unroll
        for (int k = 0; k < HC_MAX_NH; ++k) {
            if (k < nh) {
                const float c = comb[((size_t)t * nh + k) * nh + i];
                acc.x = fadd(acc.x, fmul(c, r[k].x));
                acc.y = fadd(acc.y, fmul(c, r[k].y));
                acc.z = fadd(acc.z, fmul(c, r[k].z));
                acc.w = fadd(acc.w, fmul(c, r[k].w));
            }
        }
        *reinterpret_cast<float4*>(out + ((size_t)t * nh + i) * h + j) = acc;
    }
}

int launch_rmsnorm(const float* x, const float* w, float eps, float* out, int n, int dim, hipStream_t st) {
    if (n == 0) return FERRITE_OK;
    const bool vec4 = (dim & 3) == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) |
                                           reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    // beyond ~1000 rows the chip is full either way and one wave per row wastes no idle waves (4096 rows: 62 against 66 us)
    if (vec4 && dim <= RN_ROW_MAX && n <= 1024) {
        const size_t lds = ((size_t)((dim + 255) & ~255) + 4) * sizeof(float);
        if (dim <= 1024) rmsnorm_row_kernel<1><<<n, 256, lds, st>>>(x, w, eps, out, dim);
        else if (dim <= 2048) rmsnorm_row_kernel<2><<<n, 256, lds, st>>>(x, w, eps, out, dim);
        else if (dim <= 4096) rmsnorm_row_kernel<4><<<n, 256, lds, st>>>(x, w, eps, out, dim);
        else rmsnorm_row_kernel<8><<<n, 256, lds, st>>>(x, w, eps, out, dim);
    } else {
        rmsnorm_kernel<<<n, 64, 0, st>>>(x, w, eps, out, dim);
    }
    return check_launch("rmsnorm");
}

int launch_hc_post(const float* x, const float* residual, const float* post, const float* comb, float* out, int s,
                   int nh, int h, hipStream_t st) {
    if (s == 0) return FERRITE_OK;
    dim3 grid((h / 4 + 255) / 256, s);
    hc_post_kernel<<<grid, 256, 0, st>>>(x, residual, post, comb, out, nh, h);
    return check_launch("hc_post");
}

}  // namespace fe

using namespace fe;

extern "C" int ferrite_rmsnorm_f32(const float* x, const float* w, float eps, float* out, int n, int dim,
                                   ferrite_stream_t stream) {
    if (!x || !w || !out || n < 0 || dim <= 0) return FERRITE_ERR_INVALID_ARG;
    if (n > 0x7fffffff / 2) return FERRITE_DECLINED;
    return launch_rmsnorm(x, w, eps, out, n, dim, as_stream(stream));
}

extern "C" int ferrite_hc_post_f32(const float* x, const float* residual, const float* post, const float* comb,
                                   float* out, int s, int nh, int h, ferrite_stream_t stream) {
    if (!x || !residual || !post || !comb || !out || s < 0 || nh <= 0 || h <= 0) return FERRITE_ERR_INVALID_ARG;
    if (nh > HC_MAX_NH || h % 4 != 0 || s > 65535) return FERRITE_DECLINED;
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(residual) | reinterpret_cast<uintptr_t>(out)) & 15)
        return FERRITE_ERR_INVALID_ARG;
    return launch_hc_post(x, residual, post, comb, out, s, nh, h, as_stream(stream));
}
