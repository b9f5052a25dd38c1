// Weight-streaming ("direct") MFMA GEMM for A [M,K] x B [N,K]^T with K-contiguous operands.
//
// One workgroup owns a 16*MT x 16 output tile; its NW waves split K by interleaved 128-byte
// steps, read their MFMA fragments straight from global memory (every byte of B is read by
// exactly one wave, 32 contiguous bytes per lane, a full 128-byte line per matrix row) and
// reduce through LDS.  This is the shape that wins when M is small and the GEMM is bound by
// streaming B from HBM; for large M the LDS-tiled kernels take over.
//
// The same kernel serves the grouped (per-expert segment) GEMM: a tile then first locates its
// segment from seg_indptr.
#pragma once
#include "common.hpp"

namespace llmk {

enum : int { K_FP8_BLOCK = 0, K_I8_BLOCK = 1, K_I8_ROWCOL = 2, K_F16 = 3, K_BF16 = 4 };

__device__ __forceinline__ float ld_scale(const void* p, int64_t i, int dt) {
    if (dt == LLMK_F32) return ((const float*)p)[i];
    if (dt == LLMK_F16) return f16_to_f32(((const unsigned short*)p)[i]);
    return bf16_to_f32(((const unsigned short*)p)[i]);
}

__device__ __forceinline__ void st_out(void* p, int64_t i, float v, int dt) {
    if (dt == LLMK_F32) ((float*)p)[i] = v;
    else if (dt == LLMK_F16) ((unsigned short*)p)[i] = f32_to_f16(v);
    else ((unsigned short*)p)[i] = f32_to_bf16(v);
}

__device__ __forceinline__ v8i ld32(const uint8_t* p) {
    const v4i* q = (const v4i*)p;
    v4i lo = q[0], hi = q[1];
    v8i r;
    r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
    r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
    return r;
}

// product of one 32-byte-per-lane K step, returned as fp32 (exact for the integer kinds)
template <int KIND>
__device__ __forceinline__ v4f step_dot(const v8i& a, const v8i& b) {
    const v4f z = {0.f, 0.f, 0.f, 0.f};
    if constexpr (KIND == K_FP8_BLOCK) {
        return mfma_fp8_16x16x128(a, b, z);
    } else if constexpr (KIND == K_I8_BLOCK || KIND == K_I8_ROWCOL) {
        v4i zi = {0, 0, 0, 0};
        v4i a0 = {a[0], a[1], a[2], a[3]}, a1 = {a[4], a[5], a[6], a[7]};
        v4i b0 = {b[0], b[1], b[2], b[3]}, b1 = {b[4], b[5], b[6], b[7]};
        v4i t = mfma_i8_16x16x64(a0, b0, zi);
        t = mfma_i8_16x16x64(a1, b1, t);
        v4f r = {(float)t[0], (float)t[1], (float)t[2], (float)t[3]};
        return r;
    } else {
        return z;
    }
}

struct DirectArgs {
    const uint8_t* a;      // [M, K] elements of ESZ bytes
    const uint8_t* b;      // [N, K] or [E, N, K]
    void* c;               // [M, N] c_dtype (may be null for ROWCOL when only c_i32 wanted)
    int32_t* c_i32;        // ROWCOL raw accumulators or null
    const void* a_s;       // block kinds: [M, K/128]; rowcol: fp32 [M]
    const void* b_s;       // block kinds: [(E,) ceil(N/128), K/128]; rowcol: fp32 [N]
    const int64_t* seg_indptr;      // grouped only
    const int64_t* weight_indices;  // grouped only
    int c_dtype, s_dtype;
    int M, N, K, E;
};

template <int KIND, int MT, int NW, bool GROUPED>
__global__ __launch_bounds__(NW * 64) void gemm_direct_kernel(DirectArgs p) {
    constexpr bool HALF = (KIND == K_F16 || KIND == K_BF16);
    constexpr int ESZ = HALF ? 2 : 1;
    constexpr int KSTEP = 128 / ESZ;          // elements covered by one 128-byte step
    constexpr bool BLOCKSCALE = (KIND == K_FP8_BLOCK || KIND == K_I8_BLOCK);
    extern __shared__ float red[];            // [NW][MT][64][4]

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int K = p.K, N = p.N;
    const int steps = K / KSTEP;

    int m_start, m_end;
    const uint8_t* bbase = p.b;
    int64_t bs_off = 0;
    if constexpr (GROUPED) {
        // locate the segment that owns m-tile blockIdx.y
        int tile = blockIdx.y, e = 0, cum = 0;
        int64_t s0 = p.seg_indptr[0];
        bool found = false;
        for (; e < p.E; ++e) {
            int64_t s1 = p.seg_indptr[e + 1];
            int t = (int)((s1 - s0 + 16 * MT - 1) / (16 * MT));
            if (tile < cum + t) { found = true; m_start = (int)s0 + (tile - cum) * 16 * MT; m_end = min((int)s1, m_start + 16 * MT); break; }
            cum += t;
            s0 = s1;
        }
        if (!found) return;
        const int64_t widx = p.weight_indices ? p.weight_indices[e] : e;
        bbase += widx * (int64_t)N * K * ESZ;
        bs_off = widx * (int64_t)((N + 127) / 128) * steps;
    } else {
        m_start = blockIdx.y * 16 * MT;
        m_end = min(p.M, m_start + 16 * MT);
    }

    const int nrow = min(n0 + r, N - 1);
    const uint8_t* bp = bbase + ((int64_t)nrow * K) * ESZ + 32 * g;
    const uint8_t* ap[MT];
    int srow[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int arow = min(m_start + 16 * mt + r, m_end - 1);
        ap[mt] = p.a + ((int64_t)arow * K) * ESZ + 32 * g;
#pragma unroll
        for (int i = 0; i < 4; ++i) srow[mt][i] = min(m_start + 16 * mt + 4 * g + i, m_end - 1);
    }

    v4f acc[MT];
    v4i acci[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) { acc[mt] = (v4f){0.f, 0.f, 0.f, 0.f}; acci[mt] = (v4i){0, 0, 0, 0}; }
    const int64_t bs_row = bs_off + (int64_t)(n0 / 128) * steps;

#pragma unroll 2
    for (int ks = wave; ks < steps; ks += NW) {
        const v8i b = ld32(bp + (int64_t)ks * 128);
        float bs = 1.f;
        if constexpr (BLOCKSCALE) bs = ld_scale(p.b_s, bs_row + ks, p.s_dtype);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const v8i a = ld32(ap[mt] + (int64_t)ks * 128);
            if constexpr (BLOCKSCALE) {
                const v4f t = step_dot<KIND>(a, b);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float as = ld_scale(p.a_s, (int64_t)srow[mt][i] * steps + ks, p.s_dtype);
                    acc[mt][i] += t[i] * (as * bs);
                }
            } else if constexpr (KIND == K_I8_ROWCOL) {
                v4i a0 = {a[0], a[1], a[2], a[3]}, a1 = {a[4], a[5], a[6], a[7]};
                v4i b0 = {b[0], b[1], b[2], b[3]}, b1 = {b[4], b[5], b[6], b[7]};
                acci[mt] = mfma_i8_16x16x64(a0, b0, acci[mt]);
                acci[mt] = mfma_i8_16x16x64(a1, b1, acci[mt]);
            } else if constexpr (KIND == K_F16) {
                v8h a0, a1, b0, b1;
                __builtin_memcpy(&a0, &a, 16); __builtin_memcpy(&a1, ((const char*)&a) + 16, 16);
                __builtin_memcpy(&b0, &b, 16); __builtin_memcpy(&b1, ((const char*)&b) + 16, 16);
                acc[mt] = mfma_f16_16x16x32(a0, b0, acc[mt]);
                acc[mt] = mfma_f16_16x16x32(a1, b1, acc[mt]);
            } else {
                v8bf a0, a1, b0, b1;
                __builtin_memcpy(&a0, &a, 16); __builtin_memcpy(&a1, ((const char*)&a) + 16, 16);
                __builtin_memcpy(&b0, &b, 16); __builtin_memcpy(&b1, ((const char*)&b) + 16, 16);
                acc[mt] = mfma_bf16_16x16x32(a0, b0, acc[mt]);
                acc[mt] = mfma_bf16_16x16x32(a1, b1, acc[mt]);
            }
        }
    }

    // cross-wave reduction of the K split; integer accumulators travel as raw bits
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        float* dst = red + ((wave * MT + mt) * 64 + lane) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            dst[i] = (KIND == K_I8_ROWCOL) ? __int_as_float(acci[mt][i]) : acc[mt][i];
    }
    __syncthreads();
    for (int o = threadIdx.x; o < MT * 256; o += NW * 64) {
        const int mt = o >> 8, row16 = (o & 255) >> 4, col = o & 15;
        const int src = (mt * 64 + (row16 >> 2) * 16 + col) * 4 + (row16 & 3);
        const int m = m_start + 16 * mt + row16, n = n0 + col;
        if (m >= m_end || n >= N) continue;
        if constexpr (KIND == K_I8_ROWCOL) {
            int s = 0;
#pragma unroll
            for (int w = 0; w < NW; ++w) s += __float_as_int(red[w * MT * 256 + src]);
            if (p.c_i32) p.c_i32[(int64_t)m * N + n] = s;
            if (p.c) st_out(p.c, (int64_t)m * N + n, (float)s * ((const float*)p.a_s)[m] * ((const float*)p.b_s)[n], p.c_dtype);
        } else {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) s += red[w * MT * 256 + src];
            st_out(p.c, (int64_t)m * N + n, s, p.c_dtype);
        }
    }
}

template <int KIND, bool GROUPED>
int launch_direct(const DirectArgs& p, int max_rows_per_segment_hint, hipStream_t stream, const char* name) {
    // m-tiles per workgroup: 1 for decode-sized M, up to 4 otherwise
    const int M = p.M;
    const int mt = (max_rows_per_segment_hint <= 16) ? 1 : (max_rows_per_segment_hint <= 32 ? 2 : 4);
    constexpr int NW = 8;
    dim3 block(NW * 64);
    auto tiles = [&](int rows) { return (rows + 16 * mt - 1) / (16 * mt); };
    dim3 grid((unsigned)((p.N + 15) / 16), (unsigned)(GROUPED ? tiles(M) + p.E : tiles(M)));
    if (grid.y == 0 || grid.x == 0) return LLMK_OK;
    const size_t smem = (size_t)NW * mt * 256 * sizeof(float);
    if (mt == 1) gemm_direct_kernel<KIND, 1, NW, GROUPED><<<grid, block, smem, stream>>>(p);
    else if (mt == 2) gemm_direct_kernel<KIND, 2, NW, GROUPED><<<grid, block, smem, stream>>>(p);
    else gemm_direct_kernel<KIND, 4, NW, GROUPED><<<grid, block, smem, stream>>>(p);
    LLMK_CHECK_LAUNCH(name);
    return LLMK_OK;
}

}  // namespace llmk
