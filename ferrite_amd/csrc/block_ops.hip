// The steps on either side of the MoE FFN inside a decoder layer (crates/ferrite-exec/src/lib.rs:487-492):
// rmsnorm(post_attention_layernorm) in front of it and the hyper-connection update hc_post behind it, each
// reproducing the reference's f32 evaluation order bit for bit, and the three of them as one call.
#include <hip/hip_runtime.h>

#include "internal.hpp"
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
        // batches of eight 16-byte reads, one counted wait per batch (LDS returns in order: lgkmcnt(8) = everything
        // but the batch just issued), 32 dependent adds per batch; without this the chain stalls on every read
        const float4* s4 = reinterpret_cast<const float4*>(sq);
        const int nb = len4 / 32;   // full batches
        float4 r[2][8];
        if (nb > 0) {
#pragma unroll
            for (int j = 0; j < 8; ++j) r[0][j] = s4[j];
        }
        for (int b = 0; b < nb; b += 2) {
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int bb = b + half;
                if (bb < nb) {
                    if (bb + 1 < nb) {
#pragma unroll
                        for (int j = 0; j < 8; ++j) r[half ^ 1][j] = s4[(bb + 1) * 8 + j];
                        __builtin_amdgcn_sched_barrier(0);
                        __builtin_amdgcn_s_waitcnt(0xC87F);
                    } else {
                        __builtin_amdgcn_sched_barrier(0);
                        __builtin_amdgcn_s_waitcnt(0xC07F);
                    }
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const float4 p = r[half][j];
                        ss = fadd(ss, p.x);
                        ss = fadd(ss, p.y);
                        ss = fadd(ss, p.z);
                        ss = fadd(ss, p.w);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        for (int j = nb * 8; j < len4 / 4; ++j) {
            const float4 p = s4[j];
            ss = fadd(ss, p.x);
            ss = fadd(ss, p.y);
            ss = fadd(ss, p.z);
            ss = fadd(ss, p.w);
        }
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
    rmsnorm_kernel<<<n, 64, 0, st>>>(x, w, eps, out, dim);
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
