// Shared device helpers for the gfx950 (CDNA4, wave64) kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <atomic>

#include "../../include/llmk.h"

typedef int      v2i  __attribute__((ext_vector_type(2)));
typedef int      v4i  __attribute__((ext_vector_type(4)));
typedef int      v8i  __attribute__((ext_vector_type(8)));
typedef float    v2f  __attribute__((ext_vector_type(2)));
typedef float    v4f  __attribute__((ext_vector_type(4)));
typedef _Float16 v2h  __attribute__((ext_vector_type(2)));
typedef _Float16 v4h  __attribute__((ext_vector_type(4)));
typedef _Float16 v8h  __attribute__((ext_vector_type(8)));
typedef __bf16   v8bf __attribute__((ext_vector_type(8)));
typedef unsigned short v8us __attribute__((ext_vector_type(8)));

#define LLMK_WAVE 64

// ------------------------------------------------------------------ error plumbing (host)
void llmk_set_error(const char* fmt, ...);

#define LLMK_FAIL(code, ...)            \
    do {                                \
        llmk_set_error(__VA_ARGS__);    \
        return (code);                  \
    } while (0)

#define LLMK_CHECK_LAUNCH(name)                                              \
    do {                                                                     \
        hipError_t e__ = hipGetLastError();                                  \
        if (e__ != hipSuccess)                                               \
            LLMK_FAIL(LLMK_ERR_LAUNCH, "%s: launch failed: %s", (name),      \
                      hipGetErrorString(e__));                               \
    } while (0)

// ------------------------------------------------------------------ scalar conversions
__device__ __forceinline__ float bf16_to_f32(unsigned short h) {
    return __uint_as_float(((unsigned)h) << 16);
}
// round-to-nearest-even fp32 -> bf16 (NaN kept quiet)
// round-to-nearest-even conversions on the hardware converters of gfx950 (v_cvt_pk_bf16_f32, v_cvt_pk_f16_f32)
__device__ __forceinline__ unsigned short f32_to_bf16(float f) {
    const __bf16 v = (__bf16)f;
    unsigned short h;
    __builtin_memcpy(&h, &v, 2);
    return h;
}
// two floats -> one dword of two 16-bit values (a in the low half)
__device__ __forceinline__ unsigned pack_bf16x2(float a, float b) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    const bf2 v = __builtin_convertvector((f2){a, b}, bf2);
    unsigned u;
    __builtin_memcpy(&u, &v, 4);
    return u;
}
__device__ __forceinline__ unsigned pack_f16x2(float a, float b) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    const h2 v = __builtin_convertvector((f2){a, b}, h2);
    unsigned u;
    __builtin_memcpy(&u, &v, 4);
    return u;
}
__device__ __forceinline__ float f16_to_f32(unsigned short h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}
// Keeps an fp32 value as computed.  Without it the compiler folds an fp32 multiply and the conversion of its
// result to fp16 into one v_fma_mixlo_f16, which rounds the exact product once; an operator defined as
// "multiply in fp32, then cast" rounds twice, and the two differ by an fp16 ulp where the fp32 product lands
// on a tie.  The fused form also adds +0, so a product of -0 comes out as +0.
__device__ __forceinline__ float keep_f32(float v) {
    asm volatile("" : "+v"(v));
    return v;
}
__device__ __forceinline__ unsigned short f32_to_f16(float f) {
    _Float16 v = (_Float16)f;   // v_cvt_f16_f32, RNE
    unsigned short h;
    __builtin_memcpy(&h, &v, 2);
    return h;
}

// element load as fp32 for the three float storage types (dtype codes of llmk.h)
template <int DT> struct FloatIO;
template <> struct FloatIO<LLMK_F32> {
    typedef float T;
    static __device__ __forceinline__ float ld(const void* p, int64_t i) { return ((const float*)p)[i]; }
    static __device__ __forceinline__ void st(void* p, int64_t i, float v) { ((float*)p)[i] = v; }
};
template <> struct FloatIO<LLMK_F16> {
    typedef unsigned short T;
    static __device__ __forceinline__ float ld(const void* p, int64_t i) { return f16_to_f32(((const unsigned short*)p)[i]); }
    // the value as the caller computed it in fp32, then one conversion (see keep_f32)
    static __device__ __forceinline__ void st(void* p, int64_t i, float v) { ((unsigned short*)p)[i] = f32_to_f16(keep_f32(v)); }
};
template <> struct FloatIO<LLMK_BF16> {
    typedef unsigned short T;
    static __device__ __forceinline__ float ld(const void* p, int64_t i) { return bf16_to_f32(((const unsigned short*)p)[i]); }
    static __device__ __forceinline__ void st(void* p, int64_t i, float v) { ((unsigned short*)p)[i] = f32_to_bf16(v); }
};

#define LLMK_DISPATCH_FLOAT(dt, NAME, ...)                                   \
    switch (dt) {                                                            \
        case LLMK_F32:  { constexpr int NAME = LLMK_F32;  __VA_ARGS__; break; } \
        case LLMK_F16:  { constexpr int NAME = LLMK_F16;  __VA_ARGS__; break; } \
        case LLMK_BF16: { constexpr int NAME = LLMK_BF16; __VA_ARGS__; break; } \
        default: LLMK_FAIL(LLMK_ERR_DTYPE, "unsupported float dtype code %d", (int)(dt)); \
    }

// ------------------------------------------------------------------ wave reductions
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, 64));
    return v;
}

// ------------------------------------------------------------------ MFMA wrappers (gfx950)
// 16x16 tiles.  Lane l: r = l & 15 selects the A row / B column, g = l >> 4 the K slice.
// D layout: lane holds D[4*g + i][r], i = 0..3.
__device__ __forceinline__ v4f mfma_fp8_16x16x128(v8i a, v8i b, v4f c) {
    // unscaled v_mfma_f32_16x16x128_f8f6f4, A and B format 0 = OCP e4m3
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}
__device__ __forceinline__ v4i mfma_i8_16x16x64(v4i a, v4i b, v4i c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ v4f mfma_f16_16x16x32(v8h a, v8h b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ v4f mfma_bf16_16x16x32(v8bf a, v8bf b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

static inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Compute units of MI355X: the tile kernels plan their launches in rounds of this many workgroups (one per CU).
// The plans stay correct on a device with another count (every tile is still computed exactly once); the
// launchers only take the K split of a short last round when the device really has this many.
constexpr int LLMK_CUS = 256;
// compute units of the current device (0 if the query fails); cached per process
static inline int llmk_device_cus() {
    static std::atomic<int> cache{0};
    int cus = cache.load(std::memory_order_relaxed);
    if (cus == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 0)
            cus = 0;
        cache.store(cus, std::memory_order_relaxed);
    }
    return cus;
}

// ------------------------------------------------------------------ one-time launch set-up (host)
// Opt a kernel into more than 64 KB of dynamic LDS, once per device.  `done` is a bit mask of the device
// ordinals already configured (one static mask per launch site); the call is idempotent, so two threads that
// race here merely both make it.
static inline int llmk_reserve_lds(const void* kern, int bytes, std::atomic<uint64_t>& done, const char* name) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) LLMK_FAIL(LLMK_ERR_LAUNCH, "%s: hipGetDevice: %s", name, hipGetErrorString(e));
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return LLMK_OK;
    e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) LLMK_FAIL(LLMK_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", name, bytes, hipGetErrorString(e));
    done.fetch_or(bit, std::memory_order_release);
    return LLMK_OK;
}
