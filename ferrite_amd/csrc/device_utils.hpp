// Device-side helpers shared by several translation units.
#pragma once
#include <hip/hip_runtime.h>

#include "numerics.hpp"

namespace fe {

// Activation scales are kept in the order the MFMA scale operand wants them: the e8m0 byte of the 32-wide k
// block b (k step kt = b/4, quarter g = b%4) sits at byte scale_pos(b) of its row, so that lane (column, g)
// reads the four k steps kt4*4 .. kt4*4+3 of its quarter as one dword at 16*kt4 + 4*g and selects the step
// with op_sel.  Rows are scale_pitch(K) bytes long.
__host__ __device__ __forceinline__ int scale_pos(int b) {
    const int kt = b >> 2, g = b & 3;
    return (kt >> 2) * 16 + g * 4 + (kt & 3);
}
__host__ __device__ __forceinline__ int scale_pitch(int K) { return ((K / 128 + 3) / 4) * 16; }

// Four floats to four packed e4m3 codes (byte i = value i) with the hardware converter (round to nearest even),
// made to agree with e4m3_encode(): magnitudes are clamped to 448 first, and the reference's subnormal rule
// (quant.rs:98-124: |x| in [7.5, 8) * 2^-9 encodes as 7, not as the smallest normal) is applied by moving such
// values onto 7 * 2^-9 before the conversion.  Anything that is not <= 448 in magnitude, NaN included, becomes
// +-448 as in e4m3_encode().
__device__ __forceinline__ float e4m3_prepare(float x) {
    const float ax = fabsf(x);
    x = (ax >= 0x1.ep-7f && ax < 0x1p-6f) ? copysignf(0x1.cp-7f, x) : x;
    return ax <= 448.0f ? x : copysignf(448.0f, x);
}
__device__ __forceinline__ uint32_t e4m3_encode4_hw(float a, float b, float c, float d) {
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(e4m3_prepare(a), e4m3_prepare(b), 0, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(e4m3_prepare(c), e4m3_prepare(d), w, true);
    return (uint32_t)w;
}

// Clamped SwiGLU (cpu.rs:192-201) for the MFMA mode, whose results are rounded to e4m3 right afterwards: the
// hardware exponential and reciprocal (a few ulp) instead of the bit-exact expf and division of swiglu_ref().
__device__ __forceinline__ float swiglu_fast(float g, float u, float limit) {
    // compare-and-select like swiglu_ref (cpu.rs:192-201), not fminf / fmaxf: those return the non-NaN operand and
    // would turn a NaN accumulator into +-limit
    const float gi = g > limit ? limit : g;
    const float ui = u < -limit ? -limit : (u > limit ? limit : u);
    return gi * __builtin_amdgcn_rcpf(1.0f + __expf(-gi)) * ui;
}

// 32 consecutive f32 / bf16 values (32- / 16-byte aligned) into registers.
template <typename XT>
__device__ __forceinline__ void load_block32(const XT* __restrict__ src, float (&v)[32]) {
    if constexpr (sizeof(XT) == 4) {
        const float4* p = reinterpret_cast<const float4*>(src);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float4 t = p[i];
            v[4 * i] = t.x; v[4 * i + 1] = t.y; v[4 * i + 2] = t.z; v[4 * i + 3] = t.w;
        }
    } else {
        const uint4* p = reinterpret_cast<const uint4*>(src);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint4 t = p[i];
            uint32_t wds[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[8 * i + 2 * j] = u2f(wds[j] << 16);          // bf16 -> f32 is exact
                v[8 * i + 2 * j + 1] = u2f(wds[j] & 0xffff0000u);
            }
        }
    }
}

// act_quant_fp8 of one block of 32 values held in registers (crates/ferrite-models/src/dsv41/quant.rs:190-214,
// power-of-two scale): 32 e4m3 codes to q (32-byte aligned) and the e8m0 scale byte as the return value.
// kResidual: v is replaced by what the codes leave over, v - decode(code) * scale (one f32 multiply by a power of
// two and one f32 subtraction per value), the input of the second term of a two-term quantisation.
template <bool kResidual>
__device__ __forceinline__ uint32_t encode_block32(float (&v)[32], uint8_t* __restrict__ q) {
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(v[i]));
    const uint32_t sb = block_scale_e8m0(amax);
    const float inv = u2f((254u - sb) << 23);   // 2^(127 - sb): exact reciprocal of the power-of-two scale
    const float sc = u2f(sb << 23);
    uint32_t out[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        out[i] = e4m3_encode4_hw(v[4 * i] * inv, v[4 * i + 1] * inv, v[4 * i + 2] * inv, v[4 * i + 3] * inv);
        if constexpr (kResidual) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                v[4 * i + j] = fadd(v[4 * i + j], -fmul(e4m3_decode((out[i] >> (8 * j)) & 0xffu), sc));
        }
    }
    uint4* o = reinterpret_cast<uint4*>(q);
    o[0] = make_uint4(out[0], out[1], out[2], out[3]);
    o[1] = make_uint4(out[4], out[5], out[6], out[7]);
    return sb;
}

// act_quant_fp8 of one block of 32 consecutive values in memory.
template <typename XT>
__device__ __forceinline__ uint32_t quant_block32(const XT* __restrict__ src, uint8_t* __restrict__ q) {
    float v[32];
    load_block32(src, v);
    return encode_block32<false>(v, q);
}

// Two-term quantisation of one block: x ~ decode(q1) * 2^(s1-127) + decode(q2) * 2^(s2-127), where the second
// term is act_quant_fp8 of the residual of the first.  Returns s1 | s2 << 8.
template <typename XT>
__device__ __forceinline__ uint32_t quant_block32_x2(const XT* __restrict__ src, uint8_t* __restrict__ q1,
                                                     uint8_t* __restrict__ q2) {
    float v[32];
    load_block32(src, v);
    const uint32_t s1 = encode_block32<true>(v, q1);
    const uint32_t s2 = encode_block32<false>(v, q2);
    return s1 | (s2 << 8);
}

// The left-to-right f32 sum (separately rounded adds, the reference's rmsnorm order: cpu.rs:124-143) of the n4
// float4 at s4 in LDS, continued from ss.  Every lane reads the same addresses and holds the same running sum.
// Straight-line pieces of eight batches (256 values): a batch of eight 16-byte reads is in flight while the 32
// dependent adds of the batch before it run, and nothing is in flight at the end of a piece.  With the two
// register buffers carried around a loop instead, the compiler copied one buffer into the other every iteration and
// waited for every outstanding read at the top of a batch: 15 us for 4096 values against 10 us this way.
__device__ __forceinline__ float sumsq_piece(const float4* p, float ss) {
    constexpr int NB = 8;
    float4 r[2][8];
#pragma unroll
    for (int j = 0; j < 8; ++j) r[0][j] = p[j];
#pragma unroll
    for (int g = 0; g < NB; ++g) {
        if (g + 1 < NB) {
#pragma unroll
            for (int j = 0; j < 8; ++j) r[(g + 1) & 1][j] = p[(g + 1) * 8 + j];
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0xC87F);   // lgkmcnt <= 8: everything but the batch just issued
        } else {
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0xC07F);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float4 q = r[g & 1][j];
            ss = fadd(ss, q.x);
            ss = fadd(ss, q.y);
            ss = fadd(ss, q.z);
            ss = fadd(ss, q.w);
        }
        // pins the batch's adds in front of the next batch's reads (the optimiser otherwise hoists all 64 reads of
        // the piece to its top, 256 registers) and the reads behind it
        asm volatile("" : "+v"(ss) : : "memory");
        __builtin_amdgcn_sched_barrier(0);
    }
    return ss;
}

__device__ __forceinline__ float sumsq_walk(const float4* s4, int n4, float ss) {
    const int pieces = n4 >> 6;
    for (int i = 0; i < pieces; ++i) ss = sumsq_piece(s4 + i * 64, ss);
    for (int j = pieces * 64; j < n4; ++j) {
        const float4 q = s4[j];
        ss = fadd(ss, q.x);
        ss = fadd(ss, q.y);
        ss = fadd(ss, q.z);
        ss = fadd(ss, q.w);
    }
    return ss;
}

}  // namespace fe
