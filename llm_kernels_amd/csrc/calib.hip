// Calibration kernels for the benchmark harness: what this chip sustains on the two resources the GEMM
// kernels are priced against, measured by the same process, on the same box, next to the GEMM figures.
//
//   llmk_calib_mfma  a loop of nothing but matrix instructions on random register operands: eight waves per
//                    workgroup (two per SIMD, as in the tile kernels), 32 independent accumulator tiles per wave
//                    (the 8 x 4 tile grid of the 256 x 256 kernel's wave), no memory traffic inside the loop.
//   llmk_calib_read  a read of a buffer with no arithmetic: either a linear stream, or the addresses of the
//                    weight-streaming (decode) kernels: persistent workgroups walk 16-row tiles of a matrix with
//                    4096-byte rows, the eight waves split a row by interleaved 128-byte steps, and a lane reads
//                    16-byte chunks g and g + 4 of its row (64 contiguous bytes per row and instruction).
//
// Nothing here is on the product path; the peaks the roofline divides by stay the published ones.
#include "common.hpp"

namespace {

template <int KIND>
__device__ __forceinline__ v4f calib_mma(const v8i& a, const v8i& b, v4f c) {
    if constexpr (KIND == LLMK_KIND_FP8) {
        return mfma_fp8_16x16x128(a, b, c);
    } else if constexpr (KIND == LLMK_KIND_I8) {
        v4i ci;
        __builtin_memcpy(&ci, &c, 16);
        ci = mfma_i8_16x16x64((v4i){a[0], a[1], a[2], a[3]}, (v4i){b[0], b[1], b[2], b[3]}, ci);
        __builtin_memcpy(&c, &ci, 16);
        return c;
    } else if constexpr (KIND == LLMK_KIND_F16) {
        v8h x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return mfma_f16_16x16x32(x, y, c);
    } else {
        v8bf x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return mfma_bf16_16x16x32(x, y, c);
    }
}

// operands: at least 64 KiB of random bits that are finite numbers in the operand type (the caller's business)
template <int KIND>
__global__ __launch_bounds__(512) void calib_mfma_kernel(const int* __restrict__ operands, float* __restrict__ out,
                                                         int iters, long long* __restrict__ clocks) {
    const int tid = threadIdx.x;
    v8i bf[4], af[8];
    const v8i* src = (const v8i*)operands;
#pragma unroll
    for (int j = 0; j < 4; ++j) bf[j] = src[(tid + 512 * j) & 2047];
#pragma unroll
    for (int i = 0; i < 8; ++i) af[i] = src[(tid * 3 + 512 * i + 7) & 2047];
    v4f acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = calib_mma<KIND>(bf[j], af[i], acc[i][j]);
    }
    const long long c1 = clock64(), w1 = wall_clock64();
    float r = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) r += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
    out[(size_t)blockIdx.x * blockDim.x + tid] = r;
    if (clocks && blockIdx.x == 0 && tid == 0) {
        clocks[0] = c1 - c0;          // s_memtime ticks
        clocks[1] = w1 - w0;          // s_memrealtime ticks (constant 100 MHz)
    }
}

template <int PATTERN>
__global__ __launch_bounds__(512) void calib_read_kernel(const uint8_t* __restrict__ src, int* __restrict__ sink, long long nbytes) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, g = lane >> 4;
    v4i acc = {0, 0, 0, 0};
    if constexpr (PATTERN == 0) {
        constexpr int DEPTH = 8;
        const long long stride = (long long)gridDim.x * 512 * 16;
        for (long long off = ((long long)blockIdx.x * 512 + tid) * 16; off < nbytes; off += DEPTH * stride) {
            v4i v[DEPTH];
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                const long long o = off + d * stride;
                v[d] = *(const v4i*)(src + (o < nbytes ? o : off));
            }
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) acc += v[d];
        }
    } else {
        // 16-row tiles of a matrix with 4096-byte rows (64 KiB per tile), the tile walk of gemm_direct_kernel
        const long long ntiles = nbytes >> 16;
        for (long long tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
            const uint8_t* base = src + (tile << 16) + r * 4096 + 16 * g;
            v4i v[8];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int ks = wave + 8 * u;
                v[2 * u] = *(const v4i*)(base + ks * 128);
                v[2 * u + 1] = *(const v4i*)(base + ks * 128 + 64);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) acc += v[u];
        }
    }
    if (acc[0] + acc[1] + acc[2] + acc[3] == 0x12345678) sink[0] = 1;
}

}  // namespace

extern "C" int llmk_calib_mfma(int kind, int iters, const void* operands, float* out, int workgroups, long long* clocks,
                               void* stream) {
    if (iters < 0 || workgroups <= 0 || !operands || !out) LLMK_FAIL(LLMK_ERR_ARG, "calib_mfma: bad argument");
    hipStream_t st = (hipStream_t)stream;
    const int* ops = (const int*)operands;
    switch (kind) {
        case LLMK_KIND_FP8: calib_mfma_kernel<LLMK_KIND_FP8><<<workgroups, 512, 0, st>>>(ops, out, iters, clocks); break;
        case LLMK_KIND_I8: calib_mfma_kernel<LLMK_KIND_I8><<<workgroups, 512, 0, st>>>(ops, out, iters, clocks); break;
        case LLMK_KIND_F16: calib_mfma_kernel<LLMK_KIND_F16><<<workgroups, 512, 0, st>>>(ops, out, iters, clocks); break;
        case LLMK_KIND_BF16: calib_mfma_kernel<LLMK_KIND_BF16><<<workgroups, 512, 0, st>>>(ops, out, iters, clocks); break;
        default: LLMK_FAIL(LLMK_ERR_DTYPE, "calib_mfma: kind %d", kind);
    }
    LLMK_CHECK_LAUNCH("calib_mfma");
    return LLMK_OK;
}

extern "C" int llmk_calib_read(const void* src, int64_t nbytes, int pattern, int* sink, int workgroups, void* stream) {
    if (!src || !sink || nbytes <= 0 || workgroups <= 0) LLMK_FAIL(LLMK_ERR_ARG, "calib_read: bad argument");
    if (((uintptr_t)src & 15) || nbytes % 65536) LLMK_FAIL(LLMK_ERR_ARG, "calib_read: need a 16-byte aligned buffer of whole 64 KiB tiles");
    hipStream_t st = (hipStream_t)stream;
    if (pattern == 0) calib_read_kernel<0><<<workgroups, 512, 0, st>>>((const uint8_t*)src, sink, (long long)nbytes);
    else if (pattern == 1) calib_read_kernel<1><<<workgroups, 512, 0, st>>>((const uint8_t*)src, sink, (long long)nbytes);
    else LLMK_FAIL(LLMK_ERR_ARG, "calib_read: pattern %d", pattern);
    LLMK_CHECK_LAUNCH("calib_read");
    return LLMK_OK;
}
