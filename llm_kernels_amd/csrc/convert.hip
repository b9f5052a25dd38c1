// Integer -> half-precision converters built on exponent-bias tricks instead of integer-to-float converts,
// and a one-tile-per-wave fp16 MFMA GEMM: the gfx950 counterparts of the reference's standalone study
// programs (fast_dequant/fast_dtype_convert/*.cu, fast_dequant/simple_marlin/mma_fp16.cu).
#include "common.hpp"

namespace {

// 8 nibbles of a word (nibble i at bits 4i) -> 8 fp16 values nibble - 8 in natural order.
// (q | 0x6400) is the fp16 number 1024 + q and ((q << 4) | 0x6400) is 1024 + 16 q, so one packed subtract
// resp. one packed fma yields q - 8 without any integer-to-float convert (fast_uint4_to_fp16.cu:45-97).
__device__ __forceinline__ v4i u4x8_to_f16x8(unsigned w) {
    const v2h k1032 = {(_Float16)1032.f, (_Float16)1032.f}, k16 = {(_Float16)0.0625f, (_Float16)0.0625f},
              k72 = {(_Float16)72.f, (_Float16)72.f};
    auto as_h2 = [](unsigned u) { v2h r; __builtin_memcpy(&r, &u, 4); return r; };
    auto as_u = [](v2h h) { unsigned r; __builtin_memcpy(&r, &h, 4); return r; };
    const unsigned w8 = w >> 8;
    const unsigned p04 = as_u(as_h2((w & 0x000f000fu) | 0x64006400u) - k1032);         // (n0, n4)
    const unsigned p15 = as_u(as_h2((w & 0x00f000f0u) | 0x64006400u) * k16 - k72);     // (n1, n5)
    const unsigned p26 = as_u(as_h2((w8 & 0x000f000fu) | 0x64006400u) - k1032);        // (n2, n6)
    const unsigned p37 = as_u(as_h2((w8 & 0x00f000f0u) | 0x64006400u) * k16 - k72);    // (n3, n7)
    v4i o;
    o[0] = (int)__builtin_amdgcn_perm(p15, p04, 0x05040100u);   // (n0, n1)
    o[1] = (int)__builtin_amdgcn_perm(p37, p26, 0x05040100u);   // (n2, n3)
    o[2] = (int)__builtin_amdgcn_perm(p15, p04, 0x07060302u);   // (n4, n5)
    o[3] = (int)__builtin_amdgcn_perm(p37, p26, 0x07060302u);   // (n6, n7)
    return o;
}

__global__ void u4_to_f16_kernel(const uint32_t* __restrict__ packed, unsigned short* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i * 8 >= n) return;
    const v4i o = u4x8_to_f16x8(packed[i]);
    if (i * 8 + 8 <= n) {
        *(v4i*)(out + i * 8) = o;
    } else {
        unsigned short h[8];
        __builtin_memcpy(h, &o, 16);
        for (int j = 0; i * 8 + j < n; ++j) out[i * 8 + j] = h[j];
    }
}

// bytes b -> fp16 (b - 128): 0x64bb is 1024 + b, minus 1152 (fast_uint8_to_fp16.cu)
__global__ void u8_to_f16_kernel(const uint8_t* __restrict__ in, unsigned short* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i * 8 >= n) return;
    const v2h k1152 = {(_Float16)1152.f, (_Float16)1152.f};
    auto cvt2 = [&](unsigned src, unsigned sel) {
        const unsigned u = __builtin_amdgcn_perm(0x64646464u, src, sel);
        v2h h; __builtin_memcpy(&h, &u, 4);
        h = h - k1152;
        unsigned r; __builtin_memcpy(&r, &h, 4);
        return r;
    };
    if (i * 8 + 8 <= n) {
        const uint2 s = *(const uint2*)(in + i * 8);
        v4i o;
        o[0] = (int)cvt2(s.x, 0x04010400u); o[1] = (int)cvt2(s.x, 0x04030402u);
        o[2] = (int)cvt2(s.y, 0x04010400u); o[3] = (int)cvt2(s.y, 0x04030402u);
        *(v4i*)(out + i * 8) = o;
    } else {
        for (int j = 0; i * 8 + j < n; ++j) {
            const unsigned r = cvt2(in[i * 8 + j], 0x04010400u);
            out[i * 8 + j] = (unsigned short)(r & 0xffff);
        }
    }
}

// bytes b -> bf16 (b - 128): 0x4B0000bb is the float 2^23 + b; minus (2^23 + 128), then the upper half of the
// float is the exact bf16 (fast_uint8_to_bf16.cu:26-46)
__global__ void u8_to_bf16_kernel(const uint8_t* __restrict__ in, unsigned short* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i * 8 >= n) return;
    auto cvt = [](unsigned b) {
        const float f = __uint_as_float(0x4B000000u | b) - 8388736.0f;
        return __float_as_uint(f) >> 16;
    };
    if (i * 8 + 8 <= n) {
        const uint2 s = *(const uint2*)(in + i * 8);
        const unsigned w[2] = {s.x, s.y};
        v4i o;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const unsigned src = w[k >> 1], sh = 16 * (k & 1);
            o[k] = (int)(cvt((src >> sh) & 0xff) | (cvt((src >> (sh + 8)) & 0xff) << 16));
        }
        *(v4i*)(out + i * 8) = o;
    } else {
        for (int j = 0; i * 8 + j < n; ++j) out[i * 8 + j] = (unsigned short)cvt(in[i * 8 + j]);
    }
}

// C[M,N] (fp16) = A[M,K] (fp16, row-major) x B[K,N] (fp16, row-major), one 16 x 16 tile per wave, one
// v_mfma_f32_16x16x32_f16 per 32-K step, operands gathered straight from global memory (mma_fp16.cu: one
// mma.m16n8k16 tile per warp).  Lane l: r = l & 15, g = l >> 4; A operand = A[m0 + r][k0 + 8g .. +7],
// B operand = B[k0 + 8g .. +7][n0 + r], D[i] = C[m0 + 4g + i][n0 + r].
__global__ __launch_bounds__(64) void gemm_f16_simple_kernel(const _Float16* __restrict__ A, const _Float16* __restrict__ B,
                                                             _Float16* __restrict__ C, int M, int N, int K) {
    const int lane = threadIdx.x, r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16, m0 = blockIdx.y * 16;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += 32) {
        v8h a, b;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int k = k0 + 8 * g + j;
            a[j] = (m0 + r < M && k < K) ? A[(int64_t)(m0 + r) * K + k] : (_Float16)0.f;
            b[j] = (n0 + r < N && k < K) ? B[(int64_t)k * N + n0 + r] : (_Float16)0.f;
        }
        acc = mfma_f16_16x16x32(a, b, acc);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + 4 * g + i, n = n0 + r;
        if (m < M && n < N) C[(int64_t)m * N + n] = (_Float16)acc[i];
    }
}

}  // namespace

extern "C" int llmk_convert_u4_to_f16(const uint32_t* packed, void* out, int64_t n, void* stream) {
    if (n < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "convert_u4_to_f16: negative size");
    if (n == 0) return LLMK_OK;
    if (!packed || !out) LLMK_FAIL(LLMK_ERR_ARG, "convert_u4_to_f16: null pointer");
    if ((uintptr_t)out & 15) LLMK_FAIL(LLMK_ERR_ARG, "convert_u4_to_f16: output must be 16-byte aligned");
    u4_to_f16_kernel<<<(unsigned)cdiv64(cdiv64(n, 8), 256), 256, 0, (hipStream_t)stream>>>(packed, (unsigned short*)out, n);
    LLMK_CHECK_LAUNCH("convert_u4_to_f16");
    return LLMK_OK;
}

extern "C" int llmk_convert_u8_to_f16(const uint8_t* in, void* out, int64_t n, void* stream) {
    if (n < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "convert_u8_to_f16: negative size");
    if (n == 0) return LLMK_OK;
    if (!in || !out) LLMK_FAIL(LLMK_ERR_ARG, "convert_u8_to_f16: null pointer");
    if (((uintptr_t)out & 15) || ((uintptr_t)in & 7)) LLMK_FAIL(LLMK_ERR_ARG, "convert_u8_to_f16: buffers must be 8 / 16-byte aligned");
    u8_to_f16_kernel<<<(unsigned)cdiv64(cdiv64(n, 8), 256), 256, 0, (hipStream_t)stream>>>(in, (unsigned short*)out, n);
    LLMK_CHECK_LAUNCH("convert_u8_to_f16");
    return LLMK_OK;
}

extern "C" int llmk_convert_u8_to_bf16(const uint8_t* in, void* out, int64_t n, void* stream) {
    if (n < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "convert_u8_to_bf16: negative size");
    if (n == 0) return LLMK_OK;
    if (!in || !out) LLMK_FAIL(LLMK_ERR_ARG, "convert_u8_to_bf16: null pointer");
    if (((uintptr_t)out & 15) || ((uintptr_t)in & 7)) LLMK_FAIL(LLMK_ERR_ARG, "convert_u8_to_bf16: buffers must be 8 / 16-byte aligned");
    u8_to_bf16_kernel<<<(unsigned)cdiv64(cdiv64(n, 8), 256), 256, 0, (hipStream_t)stream>>>(in, (unsigned short*)out, n);
    LLMK_CHECK_LAUNCH("convert_u8_to_bf16");
    return LLMK_OK;
}

extern "C" int llmk_gemm_f16_simple(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, void* stream) {
    if (M < 0 || N < 0 || K < 0 || M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_f16_simple: bad dimension");
    if (M == 0 || N == 0) return LLMK_OK;
    if (!c || (K && (!a || !b))) LLMK_FAIL(LLMK_ERR_ARG, "gemm_f16_simple: null pointer");
    dim3 grid((unsigned)cdiv64(N, 16), (unsigned)cdiv64(M, 16));
    gemm_f16_simple_kernel<<<grid, 64, 0, (hipStream_t)stream>>>((const _Float16*)a, (const _Float16*)b, (_Float16*)c, (int)M, (int)N, (int)K);
    LLMK_CHECK_LAUNCH("gemm_f16_simple");
    return LLMK_OK;
}
