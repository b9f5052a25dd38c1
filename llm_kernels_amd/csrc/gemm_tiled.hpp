// LDS-tiled MFMA GEMM for the compute-bound (large M) block-scaled fp8 / int8 products.
//
// Workgroup: 512 threads = 8 waves (4 along M x 2 along N), output tile 256 x 128, K step 128
// (= one scale block, one v_mfma_f32_16x16x128_f8f6f4 or two v_mfma_i32_16x16x64_i8 per 16x16 tile).
// Wave tile 64 x 64: 4 x 4 accumulator tiles (64 accumulator registers per lane), so that two waves
// share each SIMD and one wave's scale FMAs / LDS waits hide under the other's MFMAs.
// Global -> registers -> LDS with two LDS stages: the loads of K step kt+1 are in flight while
// step kt is multiplied, one barrier per step.  LDS rows are padded from 128 to 144 bytes so that
// the 16 rows a b128 read touches fall into different banks.
// Per K step the partial product of every tile is scaled by a_s[row] * b_s[column block] and
// added to the fp32 accumulator (the reference's accumulation order; the two scales are multiplied
// first, once per row, by the thread that stages them).
#pragma once
#include "gemm_direct.hpp"

namespace llmk {

constexpr int T_BM = 256, T_BN = 128, T_ROW = 144, T_THREADS = 512;
constexpr int T_A_BYTES = T_BM * T_ROW;            // 36864
constexpr int T_B_BYTES = T_BN * T_ROW;            // 18432
constexpr int T_STAGE = T_A_BYTES + T_B_BYTES + T_BM * 4;   // + the scale column of this K step
constexpr int T_LDS = 2 * T_STAGE;                 // 112640 bytes

template <int KIND, bool GROUPED, int SDT>
__global__ __launch_bounds__(T_THREADS) void gemm_tiled_kernel(DirectArgs p) {
    typedef typename ScaleIO<SDT>::Raw SRaw;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;
    const int K = p.K, N = p.N;
    const int KT = K >> 7;
    const int n0 = blockIdx.x * T_BN;

    int m_start, m_end;
    const uint8_t* bbase = p.b;
    int64_t bs_off = 0;
    if constexpr (GROUPED) {
        int tile = blockIdx.y, e = 0, cum = 0;
        int64_t s0 = p.seg_indptr[0];
        bool found = false;
        for (; e < p.E; ++e) {
            const int64_t s1 = p.seg_indptr[e + 1];
            const int t = (int)((s1 - s0 + T_BM - 1) / T_BM);
            if (tile < cum + t) { found = true; m_start = (int)s0 + (tile - cum) * T_BM; m_end = min((int)s1, m_start + T_BM); break; }
            cum += t;
            s0 = s1;
        }
        if (!found) return;
        const int64_t widx = p.weight_indices ? p.weight_indices[e] : e;
        bbase += widx * (int64_t)N * K;
        bs_off = widx * (int64_t)((N + 127) / 128) * KT;
    } else {
        m_start = blockIdx.y * T_BM;
        m_end = min(p.M, m_start + T_BM);
    }

    // ---- global -> register staging map: 8 threads cover one 128-byte row, 64 rows per pass
    const int lrow = tid >> 3, lchunk = (tid & 7) * 16;
    const uint8_t* ag[4];
    const uint8_t* bg[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) ag[i] = p.a + (int64_t)min(m_start + i * 64 + lrow, m_end - 1) * K + lchunk;
#pragma unroll
    for (int i = 0; i < 2; ++i) bg[i] = bbase + (int64_t)min(n0 + i * 64 + lrow, N - 1) * K + lchunk;
    const int64_t as_row = (int64_t)min(m_start + (tid & 255), m_end - 1) * KT;
    const int64_t bs_row = bs_off + (int64_t)blockIdx.x * KT;     // T_BN == 128: one weight-scale block per tile

    v4i ra[4], rb[2];
    SRaw raw_as = 0, raw_bs = 0;
    const SRaw* as_ptr = (const SRaw*)p.a_s + as_row;
    const SRaw* bs_ptr = (const SRaw*)p.b_s + bs_row;
    // the scale loads go first: the memory counter retires in order, and nothing may wait on them
    // before the tile loads behind them have been issued
    auto gload = [&](int kt) {
        raw_as = as_ptr[kt];
        raw_bs = bs_ptr[kt];
#pragma unroll
        for (int i = 0; i < 4; ++i) ra[i] = *(const v4i*)(ag[i] + (int64_t)kt * 128);
#pragma unroll
        for (int i = 0; i < 2; ++i) rb[i] = *(const v4i*)(bg[i] + (int64_t)kt * 128);
    };
    auto lstore = [&](int buf) {
        uint8_t* base = lds + buf * T_STAGE;
#pragma unroll
        for (int i = 0; i < 4; ++i) *(v4i*)(base + (i * 64 + lrow) * T_ROW + lchunk) = ra[i];
#pragma unroll
        for (int i = 0; i < 2; ++i) *(v4i*)(base + T_A_BYTES + (i * 64 + lrow) * T_ROW + lchunk) = rb[i];
        if (tid < T_BM) ((float*)(base + T_A_BYTES + T_B_BYTES))[tid] = ScaleIO<SDT>::cvt(raw_as) * ScaleIO<SDT>::cvt(raw_bs);
    };

    v4f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

    if (KT > 0) {
        gload(0);
        lstore(0);
    }
    __syncthreads();

    for (int kt = 0; kt < KT; ++kt) {
        const int buf = kt & 1;
        const bool more = kt + 1 < KT;
        if (more) gload(kt + 1);

        const uint8_t* As = lds + buf * T_STAGE + (wm * 64 + r) * T_ROW + 32 * g;
        const uint8_t* Bs = lds + buf * T_STAGE + T_A_BYTES + (wn * 64 + r) * T_ROW + 32 * g;
        const float* Ss = (const float*)(lds + buf * T_STAGE + T_A_BYTES + T_B_BYTES) + wm * 64 + 4 * g;
        v8i bf[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) bf[j] = ld32(Bs + j * 16 * T_ROW);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const v8i af = ld32(As + i * 16 * T_ROW);
            const v4f sa = *(const v4f*)(Ss + i * 16);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const v4f t = step_dot<KIND>(af, bf[j]);
                acc[i][j] += t * sa;
            }
        }
        if (more) lstore(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: lane holds rows 4g..4g+3 of column r in every 16x16 tile
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + wn * 64 + j * 16 + r;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int m = m_start + wm * 64 + i * 16 + 4 * g + q;
                if (m < m_end && n < N) st_out(p.c, (int64_t)m * N + n, acc[i][j][q], p.c_dtype);
            }
        }
}

template <int KIND, bool GROUPED, int SDT>
int launch_tiled_sdt(const DirectArgs& p, hipStream_t stream, const char* name) {
    static std::atomic<uint64_t> configured{0};
    auto kern = gemm_tiled_kernel<KIND, GROUPED, SDT>;
    if (int rc = llmk_reserve_lds((const void*)kern, T_LDS, configured, name)) return rc;
    const int tiles_m = GROUPED ? grouped_row_tiles(p.M, p.E, T_BM) : (p.M + T_BM - 1) / T_BM;
    dim3 grid((unsigned)((p.N + T_BN - 1) / T_BN), (unsigned)tiles_m);
    if (grid.x == 0 || grid.y == 0) return LLMK_OK;
    kern<<<grid, T_THREADS, T_LDS, stream>>>(p);
    LLMK_CHECK_LAUNCH(name);
    return LLMK_OK;
}

template <int KIND, bool GROUPED>
int launch_tiled(const DirectArgs& p, hipStream_t stream, const char* name) {
    if constexpr (KIND == K_FP8_BLOCK) {
        if (p.s_dtype != LLMK_F32) LLMK_FAIL(LLMK_ERR_DTYPE, "%s: fp8 block scales must be fp32", name);
        return launch_tiled_sdt<KIND, GROUPED, LLMK_F32>(p, stream, name);
    } else {
        switch (p.s_dtype) {
            case LLMK_F32:  return launch_tiled_sdt<KIND, GROUPED, LLMK_F32>(p, stream, name);
            case LLMK_F16:  return launch_tiled_sdt<KIND, GROUPED, LLMK_F16>(p, stream, name);
            case LLMK_BF16: return launch_tiled_sdt<KIND, GROUPED, LLMK_BF16>(p, stream, name);
            default: LLMK_FAIL(LLMK_ERR_DTYPE, "%s: s_dtype %d", name, p.s_dtype);
        }
    }
}

}  // namespace llmk
