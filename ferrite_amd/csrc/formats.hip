// MXFP4 -> f32 dequantisation and e4m3-per-32 activation quantisation.  Both are bit-exact restatements of
// crates/ferrite-models/src/dsv41/quant.rs (dequant_fp4_row32 :260-278, act_quant_fp8 :190-214) and are
// bound by HBM traffic: every thread moves 128-bit vectors.
#include "internal.hpp"
#include "device_utils.hpp"
#include "numerics.hpp"

namespace fe {

// One thread dequantises 32 columns of one row: 16 code bytes (one 128-bit load) and one scale byte in,
// 32 floats (eight 128-bit stores) out.
__global__ __launch_bounds__(256) void mxfp4_dequant_kernel(const uint8_t* __restrict__ w,
                                                            const uint8_t* __restrict__ scale, int64_t nblocks,
                                                            float* __restrict__ dst) {
    int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    uint4 c = *reinterpret_cast<const uint4*>(w + b * 16);
    float s = ue8m0_decode(scale[b]);
    uint32_t words[4] = {c.x, c.y, c.z, c.w};
    float4* o = reinterpret_cast<float4*>(dst + b * 32);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        uint32_t v = words[q];
        float4 lo, hi;
        lo.x = e2m1_decode(v & 15u) * s;         lo.y = e2m1_decode((v >> 4) & 15u) * s;
        lo.z = e2m1_decode((v >> 8) & 15u) * s;  lo.w = e2m1_decode((v >> 12) & 15u) * s;
        hi.x = e2m1_decode((v >> 16) & 15u) * s; hi.y = e2m1_decode((v >> 20) & 15u) * s;
        hi.z = e2m1_decode((v >> 24) & 15u) * s; hi.w = e2m1_decode((v >> 28) & 15u) * s;
        o[2 * q] = lo;
        o[2 * q + 1] = hi;
    }
}

// One thread quantises one block of 32 consecutive values of a row; with q2 / scale2, a second term from the
// residual of the first (quant_block32_x2).
// operand_order: scales go to scale_pos() within rows of scale_pitch(cols) bytes instead of row-major.
template <typename XT>
__global__ __launch_bounds__(256) void act_quant_kernel(const XT* __restrict__ x, int64_t nblocks, int bpr,
                                                        int operand_order, uint8_t* __restrict__ q,
                                                        uint8_t* __restrict__ scale, uint8_t* __restrict__ q2,
                                                        uint8_t* __restrict__ scale2) {
    int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const int64_t at = operand_order ? (b / bpr) * scale_pitch(bpr * 32) + scale_pos((int)(b % bpr)) : b;
    if (q2) {
        const uint32_t sb = quant_block32_x2(x + b * 32, q + b * 32, q2 + b * 32);
        scale[at] = (uint8_t)(sb & 0xffu);
        scale2[at] = (uint8_t)(sb >> 8);
    } else {
        scale[at] = (uint8_t)quant_block32(x + b * 32, q + b * 32);
    }
}

// Weights to MXFP4, one thread per block of 32 consecutive values of a row (quant.rs:217-238 with the
// power-of-two scale of :190-198 against the e2m1 maximum 6): 16 code bytes, low nibble = even column, and the
// e8m0 byte of the scale.  Nearest magnitude, a tie going to the smaller one (quant.rs:40-55 keeps the first
// candidate of a strictly-smaller search); the sign bit is set for negative inputs even when they round to zero.
FE_HD uint32_t block_scale_fp4_e8m0(float amax) {
    const uint32_t bits = f2u(fdiv(amax, 6.0f));
    const int biased = (int)((bits >> 23) & 0xFFu) + ((bits & 0x7FFFFFu) ? 1 : 0);
    return (uint32_t)(biased < 1 ? 1 : biased);
}
FE_HD uint32_t e2m1_encode(float x) {
    float a = fabsf(x);
    a = a > 6.0f ? 6.0f : a;
    const uint32_t m = (uint32_t)(a > 0.25f) + (uint32_t)(a > 0.75f) + (uint32_t)(a > 1.25f) + (uint32_t)(a > 1.75f) +
                       (uint32_t)(a > 2.5f) + (uint32_t)(a > 3.5f) + (uint32_t)(a > 5.0f);
    return m | (x < 0.0f ? 8u : 0u);
}

template <typename XT>
__global__ __launch_bounds__(256) void mxfp4_quant_kernel(const XT* __restrict__ x, int64_t nblocks,
                                                          uint8_t* __restrict__ codes, uint8_t* __restrict__ scale) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    float v[32];
    if constexpr (sizeof(XT) == 4) {
        const float4* p = reinterpret_cast<const float4*>(x + b * 32);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float4 t = p[i];
            v[4 * i] = t.x; v[4 * i + 1] = t.y; v[4 * i + 2] = t.z; v[4 * i + 3] = t.w;
        }
    } else {
        const uint4* p = reinterpret_cast<const uint4*>(x + b * 32);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint4 t = p[i];
            const uint32_t wds[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[8 * i + 2 * j] = u2f(wds[j] << 16);
                v[8 * i + 2 * j + 1] = u2f(wds[j] & 0xffff0000u);
            }
        }
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const float a = fabsf(v[i]);
        amax = a > amax ? a : amax;
    }
    const uint32_t sb = block_scale_fp4_e8m0(amax);
    const float sc = u2f(sb << 23);
    uint32_t out[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 32; ++i) out[i >> 3] |= e2m1_encode(fdiv(v[i], sc)) << (4 * (i & 7));
    *reinterpret_cast<uint4*>(codes + b * 16) = make_uint4(out[0], out[1], out[2], out[3]);
    scale[b] = (uint8_t)sb;
}

int launch_act_quant(const void* x, int x_dtype, int64_t rows, int cols, uint8_t* q, uint8_t* scale, uint8_t* q2,
                     uint8_t* scale2, int operand_order, hipStream_t st) {
    if (rows < 0 || cols < 0 || cols % 32 != 0 || (q2 == nullptr) != (scale2 == nullptr)) return FERRITE_ERR_INVALID_ARG;
    int64_t nblocks = rows * (cols / 32);
    if (nblocks == 0) return FERRITE_OK;
    unsigned grid = (unsigned)((nblocks + 255) / 256);
    if (x_dtype == FERRITE_DT_F32)
        act_quant_kernel<float><<<grid, 256, 0, st>>>((const float*)x, nblocks, cols / 32, operand_order, q, scale, q2, scale2);
    else if (x_dtype == FERRITE_DT_BF16)
        act_quant_kernel<uint16_t><<<grid, 256, 0, st>>>((const uint16_t*)x, nblocks, cols / 32, operand_order, q, scale, q2, scale2);
    else
        return FERRITE_ERR_INVALID_ARG;
    return check_launch("act_quant");
}

}  // namespace fe

using namespace fe;

extern "C" int ferrite_mxfp4_dequant(const uint8_t* w, const uint8_t* scale, int64_t rows, int64_t cols, float* dst,
                                     ferrite_stream_t stream) {
    if (rows < 0 || cols < 0 || cols % 32 != 0) return FERRITE_ERR_INVALID_ARG;
    int64_t nblocks = rows * (cols / 32);
    if (nblocks == 0) return FERRITE_OK;
    if (!w || !scale || !dst) return FERRITE_ERR_INVALID_ARG;
    if ((reinterpret_cast<uintptr_t>(w) & 15) || (reinterpret_cast<uintptr_t>(dst) & 15)) return FERRITE_DECLINED;
    mxfp4_dequant_kernel<<<(unsigned)((nblocks + 255) / 256), 256, 0, as_stream(stream)>>>(w, scale, nblocks, dst);
    return check_launch("mxfp4_dequant");
}

extern "C" int ferrite_mxfp4_quant(const void* x, int x_dtype, int64_t rows, int64_t cols, uint8_t* codes,
                                   uint8_t* scale, ferrite_stream_t stream) {
    if (rows < 0 || cols < 0 || cols % 32 != 0) return FERRITE_ERR_INVALID_ARG;
    const int64_t nblocks = rows * (cols / 32);
    if (nblocks == 0) return FERRITE_OK;
    if (!x || !codes || !scale) return FERRITE_ERR_INVALID_ARG;
    if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(codes) & 15)) return FERRITE_DECLINED;
    const unsigned grid = (unsigned)((nblocks + 255) / 256);
    if (x_dtype == FERRITE_DT_F32)
        mxfp4_quant_kernel<float><<<grid, 256, 0, as_stream(stream)>>>((const float*)x, nblocks, codes, scale);
    else if (x_dtype == FERRITE_DT_BF16)
        mxfp4_quant_kernel<uint16_t><<<grid, 256, 0, as_stream(stream)>>>((const uint16_t*)x, nblocks, codes, scale);
    else
        return FERRITE_ERR_INVALID_ARG;
    return check_launch("mxfp4_quant");
}

extern "C" int ferrite_act_quant_fp8(const void* x, int x_dtype, int64_t rows, int cols, uint8_t* q, uint8_t* scale,
                                     ferrite_stream_t stream) {
    if (rows > 0 && cols > 0 && (!x || !q || !scale)) return FERRITE_ERR_INVALID_ARG;
    if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(q) & 15)) return FERRITE_DECLINED;
    return launch_act_quant(x, x_dtype, rows, cols, q, scale, nullptr, nullptr, 0, as_stream(stream));
}

extern "C" int ferrite_act_quant_fp8_x2(const void* x, int x_dtype, int64_t rows, int cols, uint8_t* q1, uint8_t* scale1,
                                        uint8_t* q2, uint8_t* scale2, ferrite_stream_t stream) {
    if (rows > 0 && cols > 0 && (!x || !q1 || !scale1 || !q2 || !scale2)) return FERRITE_ERR_INVALID_ARG;
    if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(q1) & 15) ||
        (reinterpret_cast<uintptr_t>(q2) & 15))
        return FERRITE_DECLINED;
    return launch_act_quant(x, x_dtype, rows, cols, q1, scale1, q2, scale2, 0, as_stream(stream));
}
