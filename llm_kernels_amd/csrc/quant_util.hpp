// Helpers shared by the quantizer kernels: 8-element loads, the reference's rounding rules, e4m3 packing
// and group reductions over lanes.
#pragma once
#include "common.hpp"

namespace {

constexpr int EPL = 8;   // elements per lane in the 1 x block kernels

template <int DT>
__device__ __forceinline__ void load8(const void* p, int64_t i, float (&v)[EPL]) {
    if constexpr (DT == LLMK_F32) {
        const float4* q = (const float4*)((const float*)p + i);
        float4 a = q[0], b = q[1];
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        uint4 u = *(const uint4*)((const unsigned short*)p + i);
        unsigned w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            unsigned short lo = (unsigned short)(w[j] & 0xffff), hi = (unsigned short)(w[j] >> 16);
            v[2 * j]     = (DT == LLMK_F16) ? f16_to_f32(lo) : bf16_to_f32(lo);
            v[2 * j + 1] = (DT == LLMK_F16) ? f16_to_f32(hi) : bf16_to_f32(hi);
        }
    }
}

// 8 consecutive elements in the storage type DT (16-byte aligned for the 16-bit types, 32-byte for fp32)
template <int DT>
__device__ __forceinline__ void store8(void* p, int64_t i, const float (&v)[EPL]) {
    if constexpr (DT == LLMK_F32) {
        float4* q = (float4*)((float*)p + i);
        q[0] = make_float4(v[0], v[1], v[2], v[3]);
        q[1] = make_float4(v[4], v[5], v[6], v[7]);
    } else {
        unsigned w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            w[j] = DT == LLMK_F16 ? ((unsigned)f32_to_f16(v[2 * j]) | ((unsigned)f32_to_f16(v[2 * j + 1]) << 16))
                                  : ((unsigned)f32_to_bf16(v[2 * j]) | ((unsigned)f32_to_bf16(v[2 * j + 1]) << 16));
        *(uint4*)((unsigned short*)p + i) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

__device__ __forceinline__ float round_mode(float v, int mode) {
    // half-away: roundf is exact; half-up: floor(v + 0.5f) with the fp32 add as the reference states it
    return mode == LLMK_ROUND_HALF_AWAY ? roundf(v) : floorf(v + 0.5f);
}

__device__ __forceinline__ unsigned pack_fp8x4(float a, float b, float c, float d) {
    // saturate finite values to +-448 (comparisons leave NaN untouched), then RNE hardware convert
    auto sat = [](float x) { return x > 448.f ? 448.f : (x < -448.f ? -448.f : x); };
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(sat(a), sat(b), 0, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(sat(c), sat(d), w, true);
    return (unsigned)w;
}

// group max over the LPG lanes that share a group (LPG power of two <= 64)
template <int LPG>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
    for (int o = LPG / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
template <int LPG>
__device__ __forceinline__ float group_min(float v) {
#pragma unroll
    for (int o = LPG / 2; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, 64));
    return v;
}


// a / b from r = RN(1 / b): one product and the residual correction q - (q b - a) r, both in fma.  The
// residual is exact whenever q is within an ulp of the quotient, and the corrected value is then the rounded
// quotient (the final step of the usual fma division); in 80 M random trials over the quantisers' operand
// ranges it equalled the IEEE division every time.  Nothing may leave the normal range: callers check b
// and take the division otherwise.  A quantiser divides the 8 values of a lane by one scale, so the
// reciprocal is shared and a quotient costs three instructions instead of about ten.
// The residual is formed as its negative, q b - a, and subtracted: with a = -0 the sum q b - a is +0 and
// q - (+0) r keeps the -0 of the quotient, where q + (a - q b) r would return +0 (an e4m3 result keeps the sign
// of a zero: 0x80).
__device__ __forceinline__ float div_by(float a, float b, float r) {
    const float q = a * r;
    const float nrem = fmaf(q, b, -a);
    return fmaf(-nrem, r, q);
}
// scales whose reciprocal, products and residuals stay normal for every |a| <= 448 b that does not round to
// zero in the 8-bit result anyway
__device__ __forceinline__ bool div_by_ok(float b) { return b > 1e-30f && b < 1e30f; }

// quantise the 8 values of a lane whose group absmax is m and store them (and, from the group's first
// lane, the scale): exactly the arithmetic of the 1 x 128 activation quantizers
template <bool FP8>
__device__ __forceinline__ void quant_store8(const float (&v)[EPL], float m, void* y, int64_t off, void* s, int64_t grp,
                                             bool first_lane, int mode, bool fp8_scale_f16 = false) {
    if constexpr (FP8) {
        const float sc = m / 448.f;
        float q[EPL];
        if (div_by_ok(sc)) {
            const float r = 1.0f / sc;
#pragma unroll
            for (int j = 0; j < EPL; ++j) q[j] = div_by(v[j], sc, r);
        } else {
#pragma unroll
            for (int j = 0; j < EPL; ++j) q[j] = v[j] / sc;
        }
        uint2 o;
        o.x = pack_fp8x4(q[0], q[1], q[2], q[3]);
        o.y = pack_fp8x4(q[4], q[5], q[6], q[7]);
        *(uint2*)((uint8_t*)y + off) = o;
        if (first_lane) {
            if (fp8_scale_f16) ((unsigned short*)s)[grp] = f32_to_f16(sc);
            else ((float*)s)[grp] = sc;
        }
    } else {
        const float sc = m / 127.f;
        unsigned w[2] = {0, 0};
        const bool fast = div_by_ok(sc);
        const float r = fast ? 1.0f / sc : 0.f;
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            int qi = (int)round_mode(fast ? div_by(v[j], sc, r) : v[j] / sc, mode);
            w[j >> 2] |= ((unsigned)(qi & 0xff)) << (8 * (j & 3));
        }
        *(uint2*)((int8_t*)y + off) = make_uint2(w[0], w[1]);
        if (first_lane) ((unsigned short*)s)[grp] = f32_to_f16(sc);
    }
}

// round-trip through the storage type: the reference multiplies in the tensor dtype
// (fp16: the value is pinned first.  A product that is only converted to fp16 otherwise becomes
// v_fma_mixlo_f16(a, b, +0), and (-0) + (+0) = +0 loses the sign of a zero product, which the e4m3 quantiser
// behind the activation would store as 0x00 instead of 0x80.)
template <int DT> __device__ __forceinline__ float rnd(float v) {
    if constexpr (DT == LLMK_F16) return f16_to_f32(f32_to_f16(keep_f32(v)));
    else if constexpr (DT == LLMK_BF16) return bf16_to_f32(f32_to_bf16(v));
    else return v;
}

// 1 / (1 + e^-x).  For 16-bit tensors the result is rounded to 8 or 11 significant bits right after, so the
// hardware exp2 and reciprocal (1 ulp each in fp32) are used: large |x| gives exp2 -> inf or 0 and the
// quotient 0 or 1, as the exact expression does.  fp32 tensors keep the library routines.
template <int IDT>
__device__ __forceinline__ float sigmoid_f(float x) {
    if constexpr (IDT == LLMK_F32) return 1.0f / (1.0f + expf(-x));
    else return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}

// gated activation of one element with the reference's rounding points (activation in fp32, rounded to the
// tensor dtype, product in the tensor dtype, optional per-expert scale in the tensor dtype)
template <int IDT>
__device__ __forceinline__ float gated_act(float gv, float up, int act, bool has_scale, float scale) {
    if (act == 0) {
        gv = gv * sigmoid_f<IDT>(gv);
    } else {
        const float kAlpha = 0.7978845608028654f;
        const float u = kAlpha * (gv + 0.044715f * gv * gv * gv);
        const float th = 2.0f * sigmoid_f<IDT>(2.0f * u) - 1.0f;
        gv = 0.5f * gv * (1.0f + th);
    }
    gv = rnd<IDT>(gv);
    float r = rnd<IDT>(gv * up);
    if (has_scale) r = rnd<IDT>(r * scale);
    return r;
}

}  // namespace
