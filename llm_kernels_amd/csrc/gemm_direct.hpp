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

enum : int { K_FP8_BLOCK = 0, K_I8_BLOCK = 1, K_I8_ROWCOL = 2, K_F16 = 3, K_BF16 = 4,
             K_W4NK = 5,      // fp16 activations x 4-bit weights packed [N, K/8] (tile kernels only)
             K_W4MARLIN = 6,  // the same with weights and scales in the Marlin layout
             K_W4A8 = 7 };    // int8 activations x uint4 weights packed eight rows per word [N/8, K] with int8 zero
                              // point and scale per (row, 128-K group) and 128 x 128 block scales (tile kernels only)

__device__ __forceinline__ float ld_scale(const void* p, int64_t i, int dt) {
    if (dt == LLMK_F32) return ((const float*)p)[i];
    if (dt == LLMK_F16) return f16_to_f32(((const unsigned short*)p)[i]);
    return bf16_to_f32(((const unsigned short*)p)[i]);
}

// raw scale element (fp32 bits or 16-bit pattern) -> fp32; SDT is a dtype code known at compile time
template <int SDT> struct ScaleIO;
template <> struct ScaleIO<LLMK_F32> {
    typedef float Raw;
    static __device__ __forceinline__ float cvt(Raw v) { return v; }
};
template <> struct ScaleIO<LLMK_F16> {
    typedef unsigned short Raw;
    static __device__ __forceinline__ float cvt(Raw v) { return f16_to_f32(v); }
};
template <> struct ScaleIO<LLMK_BF16> {
    typedef unsigned short Raw;
    static __device__ __forceinline__ float cvt(Raw v) { return bf16_to_f32(v); }
};

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

// 32 bytes of a 128-byte K step for lane group g, taken as the 16-byte chunks g and g + 4 (pointer already
// offset by 16 g): the four lane groups of a row then read 64 contiguous bytes per instruction.  The K order
// inside an MFMA is free as long as both operands use the same one.
__device__ __forceinline__ v8i ld_split(const uint8_t* p) {
    const v4i lo = *(const v4i*)p, hi = *(const v4i*)(p + 64);
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
    } else if constexpr (KIND == K_I8_BLOCK || KIND == K_I8_ROWCOL || KIND == K_W4A8) {
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
    float* partial;        // split-K: fp32 [ksplit][M][N] partial sums
    int ksplit;            // 0 / 1 = no split
    int kc_steps;          // weight-streaming kernel with K ranges: 128-byte steps per range (gridDim.z ranges)
    int group;             // K_W4NK / K_W4MARLIN: K elements per fp16 group scale
    long long* clocks;     // 256-column tile kernel, calibration only: workgroup 0 leaves the s_memtime and s_memrealtime ticks it lived
    const int8_t* w4_s4;   // K_W4A8: second-level scales [N, K/128]
    const int8_t* w4_z4;   // K_W4A8: zero points [N, K/128]
    int tail_split;        // 256-column tile kernel: the tiles of a short last round are split along K (partial = scratch)    // 256-column tile kernel with the gated-activation epilogue (grouped gate / up projection, N = 2 I): c receives the
    // 1 x 128 quantised activations [M, I] in the operand type, q_scale their scales [M, I / 128]
    void* q_scale;
    int act;               // 0 = SiLU, 1 = GELU (tanh form)
    int round_mode;        // int8 rounding of the quantiser
};

// Upper bound of the row tiles of a grouped GEMM (segment ends are only known on the device): every segment
// adds at most one ragged tile, and no segment has more tiles than rows.
inline int grouped_row_tiles(int M, int E, int tile_rows) {
    const int64_t bound = ((int64_t)M + tile_rows - 1) / tile_rows + E;
    return (int)(bound < M ? bound : M);
}

// SDT: dtype code of the block scales, fixed at compile time so that a scale load is a plain typed load with
// no branch (and hence no wait for memory) between it and the loads around it.
// VEC: the weight scales of a batch are one vector load (needs four steps per batch and steps % 4 == 0).
// KR: blockIdx.z selects a K range of p.kc_steps steps (short enough for RESIDENT); the workgroup writes its
// fp32 sums to p.partial[blockIdx.z] and a second kernel adds the ranges.
template <int KIND, int MT, int NW, bool GROUPED, bool RESIDENT, int SDT, bool VEC = false, bool KR = false>
__global__ __launch_bounds__(NW * 64) void gemm_direct_kernel(DirectArgs p) {
    static_assert(!KR || (RESIDENT && !GROUPED && !VEC), "K ranges: dense, resident activations");
    typedef typename ScaleIO<SDT>::Raw SRaw;
    constexpr bool HALF = (KIND == K_F16 || KIND == K_BF16);
    constexpr int ESZ = HALF ? 2 : 1;
    constexpr int KSTEP = 128 / ESZ;          // elements covered by one 128-byte step
    constexpr bool BLOCKSCALE = (KIND == K_FP8_BLOCK || KIND == K_I8_BLOCK);
    extern __shared__ float red[];            // [NW][MT][64][4]

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform: K-step indices stay scalar
    const int r = lane & 15, g = lane >> 4;
    const int K = p.K, N = p.N;
    const int steps_all = K / KSTEP;                         // row length of the scale tables
    const int kz0 = KR ? (int)blockIdx.z * p.kc_steps : 0;   // first step of this workgroup's K range
    const int steps = KR ? min(p.kc_steps, steps_all - kz0) : steps_all;

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

    const uint8_t* ap[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int arow = min(m_start + 16 * mt + r, m_end - 1);
        ap[mt] = p.a + ((int64_t)arow * K) * ESZ + 16 * g + (int64_t)kz0 * 128;
    }
    if constexpr (KR) bbase += (int64_t)kz0 * 128;

    // A batch is U K-steps of this wave; all its loads are issued before any of them is consumed.  Steps
    // past the end are clamped to the last step and nullified.  When the whole K range of a wave fits in
    // one batch (RESIDENT), the activation fragments are loaded once and reused for every column tile the
    // workgroup processes, and the weight batch of the next tile is requested before the current tile is
    // reduced; otherwise batches are double-buffered along K.
    constexpr int U = MT == 1 ? 4 : (MT == 2 ? 2 : 1);
    struct BBatch {
        v8i b[U];
        SRaw bs[U];           // raw weight scales, converted when the batch is multiplied
    };
    struct ABatch {
        v8i a[U][MT];
    };
    const int ntiles = (N + 15) / 16;
    auto ks_of = [&](int ks0, int u, bool& valid) {
        // ks0 = first step of the batch + wave; VEC: each wave takes U consecutive steps, else waves interleave
        const int ks = VEC ? (ks0 - wave) + wave * U + u : ks0 + u * NW;
        valid = ks < steps;
        return valid ? ks : steps - 1;
    };
    auto load_b = [&](BBatch& t, int tile, int ks0) {
        const int nrow = min(tile * 16 + r, N - 1);
        const uint8_t* bp = bbase + ((int64_t)nrow * K) * ESZ + 16 * g;
        const int64_t bs_row = bs_off + (int64_t)(tile * 16 / 128) * steps_all + kz0;
        // all data loads first, then the scales as raw bits: nothing in here waits for memory
#pragma unroll
        for (int u = 0; u < U; ++u) {
            bool valid;
            const int ksc = ks_of(ks0, u, valid);
            t.b[u] = ld_split(bp + (int64_t)ksc * 128);
            if constexpr (!BLOCKSCALE) {
                if (!valid) t.b[u] = (v8i){0, 0, 0, 0, 0, 0, 0, 0};
            }
        }
        if constexpr (BLOCKSCALE) {
            if constexpr (VEC) {
                static_assert(U == 4, "one vector of four scales per batch");
                struct __attribute__((packed)) Quad { SRaw v[4]; };
                const Quad q = *(const Quad*)((const SRaw*)p.b_s + bs_row + min((ks0 - wave) + wave * U, steps - U));
#pragma unroll
                for (int u = 0; u < U; ++u) t.bs[u] = q.v[u];
            } else {
#pragma unroll
                for (int u = 0; u < U; ++u) { bool valid; t.bs[u] = ((const SRaw*)p.b_s)[bs_row + ks_of(ks0, u, valid)]; }
            }
        }
    };
    auto load_a = [&](ABatch& t, int ks0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            bool valid;
            const int ksc = ks_of(ks0, u, valid);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) t.a[u][mt] = ld_split(ap[mt] + (int64_t)ksc * 128);
        }
    };

    // activation scales of the tile rows for every K step -> LDS table
    constexpr int RB = MT == 4 ? 1 : 2;      // reduction buffers (one needs a second barrier per tile)
    float* asl = red + RB * NW * MT * 256;
    constexpr int SROWS = MT * 16;
    // The scale rows of a tile are contiguous in a_s, so table entry idx is element m_start*steps + idx
    // (entries of rows past the segment end repeat the last valid element; those rows are never stored).
    // Requested behind the first weight / activation batch and written once the whole batch has landed.
    const int n_as = BLOCKSCALE ? SROWS * steps : 0;
    const int n_as_valid = (m_end - m_start) * steps;
    const int64_t as_base = (int64_t)m_start * steps;
    int tile = blockIdx.x;
    ABatch acur, anxt;
    BBatch bcur, bnxt, bnx2;
    // Request order: activation scales, activations (both mostly L2 hits), then the first weight batch (HBM).
    // Loads return in order, so the scale table is written and published while the weights are still on
    // their way.
    SRaw stage_as[4];
    if constexpr (BLOCKSCALE) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int idx = (int)threadIdx.x + q * NW * 64;
            stage_as[q] = 0;
            if constexpr (KR) {       // the rows of a K range are not contiguous in a_s
                const int row = idx / steps, k = idx - row * steps;
                if (idx < n_as) stage_as[q] = ((const SRaw*)p.a_s)[(int64_t)min(m_start + row, m_end - 1) * steps_all + kz0 + k];
            } else {
                if (idx < n_as) stage_as[q] = ((const SRaw*)p.a_s)[as_base + min(idx, n_as_valid - 1)];
            }
        }
    }
    if (steps > 0 && tile < ntiles) {
        load_a(acur, wave);
        load_b(bcur, tile, wave);
    }
    if constexpr (BLOCKSCALE) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int idx = (int)threadIdx.x + q * NW * 64;
            if (idx < n_as) asl[idx] = ScaleIO<SDT>::cvt(stage_as[q]);
        }
        for (int idx = (int)threadIdx.x + 4 * NW * 64; idx < n_as; idx += NW * 64)   // very long K only
            asl[idx] = ScaleIO<SDT>::cvt(((const SRaw*)p.a_s)[as_base + min(idx, n_as_valid - 1)]);
        __syncthreads();
    }

    auto mul_batch = [&](const ABatch& ta, const BBatch& tb, int ks0, v4f (&acc)[MT], v4i (&acci)[MT]) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const v8i b = tb.b[u];
            bool valid;
            const int ksc = ks_of(ks0, u, valid);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const v8i a = ta.a[u][mt];
                if constexpr (BLOCKSCALE) {
                    const v4f t = step_dot<KIND>(a, b);
                    const float bs = valid ? ScaleIO<SDT>::cvt(tb.bs[u]) : 0.f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float as = asl[(mt * 16 + 4 * g + i) * steps + ksc];
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
    };

    // cross-wave reduction of the K split and store of one finished tile (alternating buffers: one barrier
    // per tile); integer accumulators travel as raw bits
    int parity = 0;
    v4f acc[MT];
    v4i acci[MT];
    auto clear_acc = [&]() {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) { acc[mt] = (v4f){0.f, 0.f, 0.f, 0.f}; acci[mt] = (v4i){0, 0, 0, 0}; }
    };
    // Per-token x per-channel kind: the scales of the outputs this thread finishes.  The row scale does not
    // depend on the tile and is read once; the column scale of a tile is requested before the tile is
    // multiplied, so that the store at its end does not wait for memory.
    constexpr int NOUT = (MT * 256 + NW * 64 - 1) / (NW * 64);      // outputs per thread and tile
    float rc_as[NOUT], rc_bs[NOUT];
    if constexpr (KIND == K_I8_ROWCOL) {
#pragma unroll
        for (int q = 0; q < NOUT; ++q) {
            const int o = (int)threadIdx.x + q * NW * 64;
            const int m = m_start + 16 * (o >> 8) + ((o & 255) >> 4);
            rc_as[q] = (p.c && o < MT * 256) ? ((const float*)p.a_s)[min(m, m_end - 1)] : 0.f;
            rc_bs[q] = 0.f;
        }
    }
    auto request_col_scales = [&](int tl) {
        if constexpr (KIND == K_I8_ROWCOL) {
            if (p.c) {
#pragma unroll
                for (int q = 0; q < NOUT; ++q) rc_bs[q] = ((const float*)p.b_s)[min(tl * 16 + ((int)threadIdx.x & 15), N - 1)];
            }
        }
    };
    auto finish = [&](int tl) __attribute__((always_inline)) {
        float* rbuf = red + (RB == 2 ? parity : 0) * NW * MT * 256;
        parity ^= 1;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            float* dst = rbuf + ((wave * MT + mt) * 64 + lane) * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                dst[i] = (KIND == K_I8_ROWCOL) ? __int_as_float(acci[mt][i]) : acc[mt][i];
        }
        __syncthreads();
        const int n0 = tl * 16;
#pragma unroll
        for (int q = 0; q < NOUT; ++q) {
            const int o = (int)threadIdx.x + q * NW * 64;
            if (o >= MT * 256) continue;
            const int mt = o >> 8, row16 = (o & 255) >> 4, col = o & 15;
            const int src = (mt * 64 + (row16 >> 2) * 16 + col) * 4 + (row16 & 3);
            const int m = m_start + 16 * mt + row16, n = n0 + col;
            if (m >= m_end || n >= N) continue;
            if constexpr (KIND == K_I8_ROWCOL) {
                int sum = 0;
#pragma unroll
                for (int w = 0; w < NW; ++w) sum += __float_as_int(rbuf[w * MT * 256 + src]);
                if (p.c_i32) p.c_i32[(int64_t)m * N + n] = sum;
                if (p.c) st_out(p.c, (int64_t)m * N + n, (float)sum * rc_as[q] * rc_bs[q], p.c_dtype);
            } else {
                float sum = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) sum += rbuf[w * MT * 256 + src];
                if constexpr (KR) p.partial[((int64_t)blockIdx.z * p.M + m) * N + n] = sum;
                else st_out(p.c, (int64_t)m * N + n, sum, p.c_dtype);
            }
        }
        if constexpr (RB == 1) __syncthreads();
        clear_acc();
    };
    clear_acc();
    const int stride = gridDim.x;

    // The batches form a ring that is never copied: a register copy of a batch whose loads are still in
    // flight would have to wait for them, which would undo the look-ahead.
    if constexpr (RESIDENT) {
        // bcur holds `tile`, bnxt is loaded here with the next tile, bnx2 inside the loop with the one after
        if (tile + stride < ntiles) load_b(bnxt, tile + stride, wave);
        auto one = [&](BBatch& cur, BBatch& fill) __attribute__((always_inline)) {
            const int t2 = tile + 2 * stride;
            request_col_scales(tile);          // ahead of the weight loads: waiting for it must not wait for them
            if (t2 < ntiles) load_b(fill, t2, wave);
            mul_batch(acur, cur, wave, acc, acci);
            finish(tile);
            tile += stride;
        };
        while (tile < ntiles) {
            one(bcur, bnx2);
            if (tile >= ntiles) break;
            one(bnxt, bcur);
            if (tile >= ntiles) break;
            one(bnx2, bnxt);
        }
    } else {
        // flattened sequence of (tile, K batch) positions, two batch pairs in ping-pong
        int ks0 = wave;
        auto one = [&](ABatch& ca, BBatch& cb, ABatch& fa, BBatch& fb) __attribute__((always_inline)) {
            const int nk = ks0 + NW * U;
            const bool more = (VEC ? (nk - wave) + wave * U : nk) < steps;   // this wave's first step of the next batch
            const int nt = more ? tile : tile + stride;
            const bool any = nt < ntiles;
            const int fk = more ? nk : wave;
            if (!more) request_col_scales(tile);   // ahead of the loads of the next batch (see above)
            if (any) { load_b(fb, nt, fk); load_a(fa, fk); }
            mul_batch(ca, cb, ks0, acc, acci);
            if (!more) finish(tile);
            tile = nt;
            ks0 = more ? nk : wave;
        };
        while (tile < ntiles) {
            one(acur, bcur, anxt, bnxt);
            if (tile >= ntiles) break;
            one(anxt, bnxt, acur, bcur);
        }
    }
}

template <int KIND, int MT, bool GROUPED, int SDT>
int launch_direct_sdt(const DirectArgs& p, hipStream_t stream, const char* name) {
    constexpr int NW = 8;
    constexpr int U = MT == 1 ? 4 : (MT == 2 ? 2 : 1);
    constexpr bool HALF = (KIND == K_F16 || KIND == K_BF16);
    constexpr bool SCALED = (KIND == K_FP8_BLOCK || KIND == K_I8_BLOCK);
    const int steps = p.K / (HALF ? 64 : 128);
    const int ntiles = (p.N + 15) / 16;
    const int mtiles = GROUPED ? grouped_row_tiles(p.M, p.E, 16 * MT) : (p.M + 16 * MT - 1) / (16 * MT);
    if (ntiles == 0 || mtiles == 0) return LLMK_OK;
    if constexpr (SCALED && !GROUPED && MT == 1) {
        if (p.kc_steps > 0) {
            // K ranges: every range fits one resident batch per wave; the caller adds the fp32 partial sums
            if (p.kc_steps > NW * U || !p.partial) LLMK_FAIL(LLMK_ERR_ARG, "%s: bad K range setup", name);
            const int nz = (steps + p.kc_steps - 1) / p.kc_steps;
            const size_t smem_r = (size_t)2 * NW * 256 * sizeof(float) + (size_t)16 * p.kc_steps * sizeof(float);
            static std::atomic<int> slots_r_cache{0};     // same value on every MI355X; recomputing it is harmless
            int slots_r = slots_r_cache.load(std::memory_order_relaxed);
            if (slots_r == 0) {
                int dev = 0, cus = 0, per_cu = 0;
                hipError_t e = hipGetDevice(&dev);
                if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
                if (e == hipSuccess)
                    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, gemm_direct_kernel<KIND, 1, NW, false, true, SDT, false, true>, NW * 64, smem_r);
                if (e != hipSuccess) LLMK_FAIL(LLMK_ERR_LAUNCH, "%s: occupancy query failed: %s", name, hipGetErrorString(e));
                slots_r = max(1, cus * max(1, per_cu));
                slots_r_cache.store(slots_r, std::memory_order_relaxed);
            }
            const int rows = mtiles * nz;
            int gx = min(ntiles, max(1, slots_r / min(rows, slots_r)));
            { const int per_wg = (ntiles + gx - 1) / gx; gx = (ntiles + per_wg - 1) / per_wg; }
            gemm_direct_kernel<KIND, 1, NW, false, true, SDT, false, true>
                <<<dim3((unsigned)gx, (unsigned)mtiles, (unsigned)nz), dim3(NW * 64), smem_r, stream>>>(p);
            LLMK_CHECK_LAUNCH(name);
            return LLMK_OK;
        }
    }
    const size_t smem = (size_t)(MT == 4 ? 1 : 2) * NW * MT * 256 * sizeof(float) + (SCALED ? (size_t)MT * 16 * steps * sizeof(float) : 0);
    if (smem > 64 * 1024) LLMK_FAIL(LLMK_ERR_SHAPE, "%s: K=%d too large for the weight-streaming kernel's scale table", name, p.K);
    // Column tiles are processed persistently by as many workgroups as are resident at once (so that every
    // workgroup streams tile after tile with its next tiles already requested), split over the m-tile rows.
    const bool resident = steps <= NW * U;
    constexpr bool CAN_VEC = SCALED && U == 4;
    // long K: consecutive steps per wave, one load for the four weight scales of a batch (measured faster at
    // K = 14336, slower at K = 4096 where the interleaved order spreads the first requests over more channels)
    const bool vec = CAN_VEC && !resident && steps % 4 == 0;
    static std::atomic<int> slots_cache[2];   // resident workgroups on the whole device, per kernel variant
    int slots[2] = {slots_cache[0].load(std::memory_order_relaxed), slots_cache[1].load(std::memory_order_relaxed)};
    if (slots[resident] == 0) {
        int dev = 0, cus = 0, per_cu = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (e == hipSuccess)
            e = resident ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, gemm_direct_kernel<KIND, MT, NW, GROUPED, true, SDT>, NW * 64, 64 * 1024)
                         : hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, gemm_direct_kernel<KIND, MT, NW, GROUPED, false, SDT>, NW * 64, 64 * 1024);
        if (e != hipSuccess) LLMK_FAIL(LLMK_ERR_LAUNCH, "%s: occupancy query failed: %s", name, hipGetErrorString(e));
        slots[resident] = max(1, cus * max(1, per_cu));
        slots_cache[resident].store(slots[resident], std::memory_order_relaxed);
    }
    int gx = min(ntiles, max(1, slots[resident] / min(mtiles, slots[resident])));
    // every workgroup the same number of column tiles (the slowest one sets the time): fewer workgroups
    // rather than a last round that only some of them take part in
    { const int per_wg = (ntiles + gx - 1) / gx; gx = (ntiles + per_wg - 1) / per_wg; }
    dim3 grid((unsigned)gx, (unsigned)mtiles), block(NW * 64);
    if constexpr (CAN_VEC) {
        if (vec) {
            gemm_direct_kernel<KIND, MT, NW, GROUPED, false, SDT, true><<<grid, block, smem, stream>>>(p);
            LLMK_CHECK_LAUNCH(name);
            return LLMK_OK;
        }
    }
    if (resident) gemm_direct_kernel<KIND, MT, NW, GROUPED, true, SDT><<<grid, block, smem, stream>>>(p);
    else gemm_direct_kernel<KIND, MT, NW, GROUPED, false, SDT><<<grid, block, smem, stream>>>(p);
    LLMK_CHECK_LAUNCH(name);
    return LLMK_OK;
}

// the scale dtype only matters for the int8 block kind (fp8 scales are fp32, the other kinds carry none)
template <int KIND, int MT, bool GROUPED>
int launch_direct_mt(const DirectArgs& p, hipStream_t stream, const char* name) {
    if constexpr (KIND == K_I8_BLOCK) {
        switch (p.s_dtype) {
            case LLMK_F32:  return launch_direct_sdt<KIND, MT, GROUPED, LLMK_F32>(p, stream, name);
            case LLMK_F16:  return launch_direct_sdt<KIND, MT, GROUPED, LLMK_F16>(p, stream, name);
            case LLMK_BF16: return launch_direct_sdt<KIND, MT, GROUPED, LLMK_BF16>(p, stream, name);
            default: LLMK_FAIL(LLMK_ERR_DTYPE, "%s: s_dtype %d", name, p.s_dtype);
        }
    } else {
        if (KIND == K_FP8_BLOCK && p.s_dtype != LLMK_F32) LLMK_FAIL(LLMK_ERR_DTYPE, "%s: fp8 block scales must be fp32", name);
        return launch_direct_sdt<KIND, MT, GROUPED, LLMK_F32>(p, stream, name);
    }
}

template <int KIND, bool GROUPED>
int launch_direct(const DirectArgs& p, int max_rows_per_segment_hint, hipStream_t stream, const char* name) {
    // m-tiles per workgroup: 1 for decode-sized M, up to 4 otherwise.  When a wave's K share fits one batch at
    // one m-tile per workgroup (activations resident in registers), 16-row workgroups side by side beat taller
    // ones that have to re-read their activations for every column tile.
    constexpr int KSTEP = (KIND == K_F16 || KIND == K_BF16) ? 64 : 128;
    if (max_rows_per_segment_hint <= 16 || p.K / KSTEP <= 32 || p.kc_steps > 0) return launch_direct_mt<KIND, 1, GROUPED>(p, stream, name);
    if (max_rows_per_segment_hint <= 32) return launch_direct_mt<KIND, 2, GROUPED>(p, stream, name);
    return launch_direct_mt<KIND, 4, GROUPED>(p, stream, name);
}

}  // namespace llmk
