// W4A16 GEMM kernels: fp16 activations x 4-bit weights dequantised in registers.
//
// nibble -> fp16 without integer->float converts: (q | 0x6400) is the fp16 number 1024 + q,
// ((q << 4) | 0x6400) is 1024 + 16 q; one packed subtract / fma gives q - 8 exactly.
#include <algorithm>
#include "gemm_wide.hpp"
#include "stream_ring.hpp"

namespace {

__device__ __forceinline__ v2h as_h2(unsigned u) { v2h r; __builtin_memcpy(&r, &u, 4); return r; }
__device__ __forceinline__ unsigned as_u32(v2h h) { unsigned r; __builtin_memcpy(&r, &h, 4); return r; }

// nibbles at bits [3:0] and [19:16] of w -> (q_lo - 8, q_hi - 8)
__device__ __forceinline__ v2h deq_lo(unsigned w) {
    const v2h k1032 = {(_Float16)1032.f, (_Float16)1032.f};
    return as_h2((w & 0x000f000fu) | 0x64006400u) - k1032;
}
// nibbles at bits [7:4] and [23:20]
__device__ __forceinline__ v2h deq_hi(unsigned w) {
    const v2h k16 = {(_Float16)0.0625f, (_Float16)0.0625f};
    const v2h k72 = {(_Float16)72.f, (_Float16)72.f};
    return as_h2((w & 0x00f000f0u) | 0x64006400u) * k16 - k72;
}

__device__ __forceinline__ v8h make8(v2h a, v2h b, v2h c, v2h d) {
    v8h r;
    r[0] = a[0]; r[1] = a[1]; r[2] = b[0]; r[3] = b[1];
    r[4] = c[0]; r[5] = c[1]; r[6] = d[0]; r[7] = d[1];
    return r;
}

// Tree reduction of per-wave accumulators through LDS; the total ends in wave 0.
template <int NW, int NACC>
__device__ __forceinline__ void reduce_waves(float (&acc)[NACC], float* buf, int wave, int lane) {
#pragma unroll
    for (int half = NW / 2; half >= 1; half >>= 1) {
        if (wave >= half && wave < 2 * half) {
            float* dst = buf + (size_t)(wave - half) * NACC * 64;
#pragma unroll
            for (int i = 0; i < NACC; ++i) dst[i * 64 + lane] = acc[i];
        }
        __syncthreads();
        if (wave < half) {
            const float* src = buf + (size_t)wave * NACC * 64;
#pragma unroll
            for (int i = 0; i < NACC; ++i) acc[i] += src[i * 64 + lane];
        }
        __syncthreads();
    }
}

// ------------------------------------------------------------------------------------------
// simple-Marlin layout.  B viewed as 16-byte units: unit ((strip * N/64) + chunk) * 32 + 4c + q
// holds, for mma lane (c = column within 8, q = k pair), word j = 16-column sub-tile j:
//   bits  3:0 (k0, c)   7:4 (k0+8, c)   11:8 (k0, c+8)   15:12 (k0+8, c+8)      k0 = 2q
//   bits 19:16 (k0+1,c) 23:20 (k0+9,c)  27:24 (k0+1,c+8) 31:28 (k0+9,c+8)
// Scales are stored per 64-column chunk as [c][2j + b] (column 16j + 8b + c).
//
// gfx950 mapping: a wave owns two chunks (128 columns).  Lane l: r = l & 15 -> c = r & 7,
// chunk half h = r >> 3; g = l >> 4 plays the role of the mma k-pair q.  One MFMA 16x16x32
// step consumes two 16-K strips; MFMA (j, b) produces columns {64(2cp+h) + 16j + 8b + c}.
// A fragment order per lane: k in {2g, 2g+1, 2g+8, 2g+9} of strip 0, then of strip 1.
// A_LDS: the activations of the workgroup's K range are staged once in LDS, already in fragment order (one
// 16-byte read per lane and step), instead of four 4-byte global loads per lane and step.
template <int MT, int NW, bool TO_WS, bool A_LDS = false>
__global__ __launch_bounds__(NW * 64) void w4a16_marlin_kernel(
    const _Float16* __restrict__ A, const v4i* __restrict__ B, const _Float16* __restrict__ S,
    _Float16* __restrict__ C, float* __restrict__ ws, int M, int N, int K, int groupsize, int steps_per_z) {
    extern __shared__ float red[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, g = lane >> 4, c = r & 7, h = r >> 3;
    const int nchunks = N >> 6;
    const int strips = K >> 4;
    const int total_steps = (strips + 1) >> 1;
    const int chunk_raw = 2 * blockIdx.x + h;
    const bool chunk_ok = chunk_raw < nchunks;
    const int chunk = chunk_ok ? chunk_raw : nchunks - 1;
    const int m0 = blockIdx.y * 16 * MT;
    const int ks_begin = blockIdx.z * steps_per_z;
    const int ks_end = min(total_steps, ks_begin + steps_per_z);

    const _Float16* arow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) arow[mt] = A + (int64_t)min(m0 + 16 * mt + r, M - 1) * K + 2 * g;

    float acc[MT * 32];
#pragma unroll
    for (int i = 0; i < MT * 32; ++i) acc[i] = 0.f;

    // LDS image of A for steps [ks_begin, ks_end): row-major over the tile rows, per step 64 bytes = four lane
    // groups x {strip 0: k 2g, 2g+1 | 2g+8, 2g+9; strip 1: the same}; rows padded by 16 bytes (bank spread).
    const int nst = max(ks_end - ks_begin, 0);
    const int rstride = nst * 64 + 16;
    uint8_t* alds = (uint8_t*)red;
    if constexpr (A_LDS) {
        const int chunks = 16 * MT * nst * 4;                // 16-byte pieces: (row, step, strip parity, k half)
        for (int idx = threadIdx.x; idx < chunks; idx += NW * 64) {
            const int row = idx / (nst * 4), rem = idx - row * (nst * 4), ks = rem >> 2, ch = rem & 3;
            const int strip = 2 * (ks_begin + ks) + (ch >> 1);
            v4i v = {0, 0, 0, 0};
            if (strip < strips) v = *(const v4i*)(A + (int64_t)min(m0 + row, M - 1) * K + strip * 16 + (ch & 1) * 8);
            uint8_t* dst = alds + row * rstride + ks * 64 + ch * 4;
#pragma unroll
            for (int q = 0; q < 4; ++q) *(int*)(dst + q * 16) = v[q];
        }
        __syncthreads();
    }

    // Batches of U steps: every load of a batch (weights, scales, activations) is issued before the first
    // one is used, with clamped indices and no branch in between, so that a batch costs one memory round
    // trip.  Steps past the end of the range multiply by a zero activation fragment.
    constexpr int U = MT == 4 ? 1 : 2;
    const v4i* bptr = B + (int64_t)chunk * 32 + 4 * c + g;
    const int64_t strip_stride = (int64_t)nchunks * 32;
    const _Float16* sptr = S + 64 * chunk + 8 * c;
    for (int ks0 = ks_begin + wave; ks0 < ks_end; ks0 += U * NW) {
        v4i w0[U], w1[U], x[U][MT];
        v8h s0[U], s1[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ks = min(ks0 + u * NW, ks_end - 1);
            const int st0 = 2 * ks, st1 = min(2 * ks + 1, strips - 1);
            w0[u] = bptr[st0 * strip_stride];
            w1[u] = bptr[st1 * strip_stride];
            s0[u] = *(const v8h*)(sptr + (int64_t)((16 * st0) / groupsize) * N);
            s1[u] = *(const v8h*)(sptr + (int64_t)((16 * st1) / groupsize) * N);
            const int o1 = 2 * ks + 1 < strips ? 8 : 0;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if constexpr (A_LDS) {
                    x[u][mt] = *(const v4i*)(alds + (16 * mt + r) * rstride + (ks - ks_begin) * 64 + g * 16);
                } else {
                    const unsigned* ap = (const unsigned*)(arow[mt] + 32 * ks);
                    x[u][mt] = (v4i){(int)ap[0], (int)ap[4], (int)ap[o1], (int)ap[o1 + 4]};
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);       // keep every load above ahead of the first use below
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ks = ks0 + u * NW;
            const bool valid = ks < ks_end, valid1 = valid && 2 * ks + 1 < strips;
            v8h a[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                a[mt] = make8(as_h2(valid ? (unsigned)x[u][mt][0] : 0u), as_h2(valid ? (unsigned)x[u][mt][1] : 0u),
                              as_h2(valid1 ? (unsigned)x[u][mt][2] : 0u), as_h2(valid1 ? (unsigned)x[u][mt][3] : 0u));
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int b = 0; b < 2; ++b) {
                    const int t = 2 * j + b;
                    const unsigned u0 = ((unsigned)w0[u][j]) >> (8 * b), u1 = ((unsigned)w1[u][j]) >> (8 * b);
                    const v2h sc0 = {s0[u][t], s0[u][t]}, sc1 = {s1[u][t], s1[u][t]};
                    const v8h bf = make8(deq_lo(u0) * sc0, deq_hi(u0) * sc0, deq_lo(u1) * sc1, deq_hi(u1) * sc1);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        v4f d = {acc[(mt * 8 + t) * 4 + 0], acc[(mt * 8 + t) * 4 + 1], acc[(mt * 8 + t) * 4 + 2], acc[(mt * 8 + t) * 4 + 3]};
                        d = mfma_f16_16x16x32(a[mt], bf, d);
                        acc[(mt * 8 + t) * 4 + 0] = d[0]; acc[(mt * 8 + t) * 4 + 1] = d[1];
                        acc[(mt * 8 + t) * 4 + 2] = d[2]; acc[(mt * 8 + t) * 4 + 3] = d[3];
                    }
                }
            }
        }
    }

    // one-barrier reduction over the waves: slot e of lane l of wave w sits at red[(w * NE + e) * 64 + l]
    constexpr int NE = MT * 32;
    if constexpr (A_LDS) __syncthreads();                    // the reduction buffer reuses the activation image
#pragma unroll
    for (int e = 0; e < NE; ++e) red[(wave * NE + e) * 64 + lane] = acc[e];
    __syncthreads();
    for (int e = wave; e < NE; e += NW) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) v += red[(w * NE + e) * 64 + lane];
        const int mt = e >> 5, t = (e >> 2) & 7, i = e & 3;
        const int m = m0 + 16 * mt + 4 * g + i;
        const int n = 64 * chunk + 16 * (t >> 1) + 8 * (t & 1) + c;
        if (chunk_ok && m < M) {
            if constexpr (TO_WS) ws[((int64_t)blockIdx.z * M + m) * N + n] = v;
            else C[(int64_t)m * N + n] = (_Float16)v;
        }
    }
}

// four outputs per thread (MN is a multiple of 64): all Z partial vectors are requested before the first add
__global__ void splitk_reduce_f16_kernel(const float* __restrict__ ws, _Float16* __restrict__ C, int64_t MN, int Z) {
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= MN) return;
    v4f s = {0.f, 0.f, 0.f, 0.f};
    int z = 0;
    for (; z + 8 <= Z; z += 8) {
        v4f t[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) t[j] = *(const v4f*)(ws + (int64_t)(z + j) * MN + i);
#pragma unroll
        for (int j = 0; j < 8; ++j) s += t[j];
    }
    for (; z < Z; ++z) s += *(const v4f*)(ws + (int64_t)z * MN + i);
    const v2h lo = {(_Float16)s[0], (_Float16)s[1]}, hi = {(_Float16)s[2], (_Float16)s[3]};
    unsigned u0, u1;
    __builtin_memcpy(&u0, &lo, 4);
    __builtin_memcpy(&u1, &hi, 4);
    *(uint2*)(C + i) = make_uint2(u0, u1);
}

// ------------------------------------------------------------------------------------------
// Marlin words -> dequantised fp16 W^T [N][K] (K contiguous), the operand layout of the tiled GEMM.
// One workgroup converts 8 strips (128 K) of one 64-column chunk: every thread expands one 16-byte unit
// (32 values, scaled in fp16 exactly as the fused kernels do), the tile is transposed through LDS and
// written as 256-byte row segments.
__global__ __launch_bounds__(256) void marlin_dequant_kernel(const v4i* __restrict__ B, const _Float16* __restrict__ S,
                                                             _Float16* __restrict__ Wt, int N, int K, int groupsize) {
    __shared__ __attribute__((aligned(16))) _Float16 tile[64][136];
    const int tid = threadIdx.x, sl = tid >> 5, ml = tid & 31, c = ml >> 2, q = ml & 3;
    const int nchunks = N >> 6, strips = K >> 4;
    const int chunk = blockIdx.x, strip = blockIdx.y * 8 + sl;
    if (strip < strips) {
        const v4i w = B[((int64_t)strip * nchunks + chunk) * 32 + ml];
        const v8h sc = *(const v8h*)(S + (int64_t)((16 * strip) / groupsize) * N + 64 * chunk + 8 * c);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const unsigned u = ((unsigned)w[j]) >> (8 * b);
                const v2h s2 = {sc[2 * j + b], sc[2 * j + b]};
                const int n = 16 * j + 8 * b + c, k = 16 * sl + 2 * q;
                *(v2h*)&tile[n][k] = deq_lo(u) * s2;
                *(v2h*)&tile[n][k + 8] = deq_hi(u) * s2;
            }
    }
    __syncthreads();
    // eight lanes write one 128-byte line of a row per instruction
    const int seg = tid & 7;
    const int k0 = blockIdx.y * 128;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const int row = pass * 32 + (tid >> 3);
#pragma unroll
        for (int x = 0; x < 2; ++x) {
            const int kl = x * 64 + seg * 8;
            if (k0 + kl < K)
                *(v8h*)(Wt + (int64_t)(64 * chunk + row) * K + k0 + kl) = *(const v8h*)&tile[row][kl];
        }
    }
}

// ------------------------------------------------------------------------------------------
// [N, K/8] layout (pack_weights_over_cols: nibble i of word w of row n is k = 8w + i) with
// scales [N, K/g].  Lane (r = column, g) loads one 16-byte unit = 32 consecutive k of its row per
// 128-K step; word j feeds MFMA j, whose fragment order is k offsets [0,4,1,5,2,6,3,7] -- the A
// fragment is permuted to the same order with v_perm_b32.
template <int MT, int NW>
__global__ __launch_bounds__(NW * 64) void w4a16_nk_kernel(
    const _Float16* __restrict__ A, const int32_t* __restrict__ B, const _Float16* __restrict__ S,
    _Float16* __restrict__ C, int M, int N, int K, int groupsize) {
    extern __shared__ float red[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16, m0 = blockIdx.y * 16 * MT;
    const int nrow = min(n0 + r, N - 1);
    const int steps = K >> 7;
    const int ngroups = K / groupsize;
    const int32_t* brow = B + (int64_t)nrow * (K >> 3) + 4 * g;
    const _Float16* srow = S + (int64_t)nrow * ngroups;
    const _Float16* arow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) arow[mt] = A + (int64_t)min(m0 + 16 * mt + r, M - 1) * K + 32 * g;

    float acc[MT * 4];
#pragma unroll
    for (int i = 0; i < MT * 4; ++i) acc[i] = 0.f;

#pragma unroll 2
    for (int ks = wave; ks < steps; ks += NW) {
        const v4i w = *(const v4i*)(brow + ks * 16);
        const int kbase = ks * 128 + 32 * g;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const _Float16 sv = srow[(kbase + 8 * j) / groupsize];
            const v2h sc = {sv, sv};
            const unsigned u = (unsigned)w[j], u8 = u >> 8;
            const v8h bf = make8(deq_lo(u) * sc, deq_hi(u) * sc, deq_lo(u8) * sc, deq_hi(u8) * sc);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const v4i x = *(const v4i*)(arow[mt] + ks * 128 + 8 * j);
                v4i y;
                y[0] = (int)__builtin_amdgcn_perm((unsigned)x[2], (unsigned)x[0], 0x05040100u);  // k0,k4
                y[1] = (int)__builtin_amdgcn_perm((unsigned)x[2], (unsigned)x[0], 0x07060302u);  // k1,k5
                y[2] = (int)__builtin_amdgcn_perm((unsigned)x[3], (unsigned)x[1], 0x05040100u);  // k2,k6
                y[3] = (int)__builtin_amdgcn_perm((unsigned)x[3], (unsigned)x[1], 0x07060302u);  // k3,k7
                v8h a;
                __builtin_memcpy(&a, &y, 16);
                v4f d = {acc[mt * 4 + 0], acc[mt * 4 + 1], acc[mt * 4 + 2], acc[mt * 4 + 3]};
                d = mfma_f16_16x16x32(a, bf, d);
                acc[mt * 4 + 0] = d[0]; acc[mt * 4 + 1] = d[1]; acc[mt * 4 + 2] = d[2]; acc[mt * 4 + 3] = d[3];
            }
        }
    }
    reduce_waves<NW, MT * 4>(acc, red, wave, lane);
    if (wave != 0) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = m0 + 16 * mt + 4 * g + i, n = n0 + r;
            if (m < M && n < N) C[(int64_t)m * N + n] = (_Float16)acc[mt * 4 + i];
        }
}

// [N, K/8] words -> dequantised fp16 W [N][K] (the operand layout of the tiled GEMM): one thread expands one
// word (8 consecutive k of a row) and stores 16 bytes.
__global__ void nk_dequant_kernel(const int32_t* __restrict__ B, const _Float16* __restrict__ S, _Float16* __restrict__ W,
                                  int64_t N, int64_t K, int groupsize) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t kw = K >> 3;
    if (idx >= N * kw) return;
    const int64_t n = idx / kw, k = (idx - n * kw) * 8;
    const unsigned w = (unsigned)B[idx], w8 = w >> 8;
    const _Float16 sv = S[n * (K / groupsize) + k / groupsize];
    const v2h sc = {sv, sv};
    const unsigned p04 = as_u32(deq_lo(w) * sc), p15 = as_u32(deq_hi(w) * sc), p26 = as_u32(deq_lo(w8) * sc), p37 = as_u32(deq_hi(w8) * sc);
    v4i o;
    o[0] = (int)__builtin_amdgcn_perm(p15, p04, 0x05040100u);
    o[1] = (int)__builtin_amdgcn_perm(p37, p26, 0x05040100u);
    o[2] = (int)__builtin_amdgcn_perm(p15, p04, 0x07060302u);
    o[3] = (int)__builtin_amdgcn_perm(p37, p26, 0x07060302u);
    *(v4i*)(W + n * K + k) = o;
}

// The same for bf16 operands: (q - 8) * s formed in fp32 and rounded once to bf16, natural k order.
__global__ void nk_dequant_bf16_kernel(const int32_t* __restrict__ B, const _Float16* __restrict__ S,
                                       unsigned short* __restrict__ W, int64_t N, int64_t K, int groupsize) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t kw = K >> 3;
    if (idx >= N * kw) return;
    const int64_t n = idx / kw, k = (idx - n * kw) * 8;
    const unsigned w = (unsigned)B[idx];
    const float sc = (float)S[n * (K / groupsize) + k / groupsize];
    v4i o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float lo = (float)((int)((w >> (8 * i)) & 15u) - 8) * sc, hi = (float)((int)((w >> (8 * i + 4)) & 15u) - 8) * sc;
        o[i] = (int)pack_bf16x2(lo, hi);
    }
    *(v4i*)(W + n * K + k) = o;
}

// Weight-streaming variant of the [N, K/8] kernel for groupsize % 128 == 0 (every 128-K step lies in one
// scale group): persistent workgroups of 8 waves walk 16-column tiles; the waves split K by interleaved
// 128-K steps in batches of U, all loads of a batch issued before its first use and the weights of the next
// two tiles requested ahead.  When a wave's K share fits one batch (RESIDENT) its activation fragments are
// loaded and permuted once and stay in registers for every tile.  The group scale multiplies the fp32
// partial of the step (one FMA per output) instead of the eight fp16 weights.
template <int MT, int NT, bool RESIDENT, bool VS = false>
__global__ __launch_bounds__(512) void w4a16_nk_stream_kernel(
    const _Float16* __restrict__ A, const int32_t* __restrict__ B, const _Float16* __restrict__ S,
    _Float16* __restrict__ C, int M, int N, int Kfull, int groupsize, int Kc, float* __restrict__ partial) {
    constexpr int NW = 8;
    constexpr int U = MT == 1 ? 4 : (MT == 2 ? 2 : 1);
    extern __shared__ float red[];                       // [2][NW][NT][MT][64][4]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, g = lane >> 4;
    // K range [k0, k0 + K) of this workgroup (gridDim.z ranges of Kc cover rows that are Kfull long; with more
    // than one range the outputs are fp32 partial sums for a summing pass)
    const int k0 = (int)blockIdx.z * Kc, K = min(Kc, Kfull - k0);
    const int steps = K >> 7, ngroups = Kfull / groupsize, kwords = Kfull >> 3;
    const int m0 = blockIdx.y * 16 * MT;
    const int ntiles = (N + 16 * NT - 1) / (16 * NT);    // a tile is NT adjacent 16-column blocks

    const _Float16* arow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) arow[mt] = A + (int64_t)min(m0 + 16 * mt + r, M - 1) * Kfull + k0 + 32 * g;

    struct BBatch {
        v4i w[NT][U];
        unsigned short s[NT][U];
        uint2 sv[NT];          // VS: the four scales of the batch as loaded (unpacked when the batch is multiplied:
                               // any arithmetic on a value still in flight would wait for it right away)
    };
    struct ABatch {
        v4i a[U][MT][4];
    };
    // step u of the batch that starts at ks0 (= first step of the batch + wave).  VS: every wave takes U
    // consecutive steps and, with 128-wide groups, fetches their four scales with one load.
    auto step_of = [&](int ks0, int u) { return VS ? (ks0 - wave) + wave * U + u : ks0 + u * NW; };
    auto clamp_step = [&](int ks) { return min(ks, steps - 1); };
    // Addresses are a wave-uniform base (tile, K step: scalar registers) plus one 32-bit offset per lane, so that
    // a load needs no 64-bit per-lane address arithmetic and no address registers that could collide with
    // the destinations of loads still in flight.  Rows past N in the last tile repeat the last row.
    auto load_b = [&](BBatch& t, int tile, int ks0) __attribute__((always_inline)) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int rowbase = (tile * NT + nt) * 16;
            const uint32_t lo = (uint32_t)min(r, N - 1 - rowbase) * (uint32_t)(kwords * 4) + 16u * (uint32_t)g;
            const char* tb = (const char*)B + ((int64_t)rowbase * kwords + (k0 >> 3)) * 4;
#pragma unroll
            for (int u = 0; u < U; ++u) t.w[nt][u] = *(const v4i*)(tb + (int64_t)clamp_step(step_of(ks0, u)) * 64 + lo);
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int rowbase = (tile * NT + nt) * 16;
            const uint32_t lo = (uint32_t)min(r, N - 1 - rowbase) * (uint32_t)(ngroups * 2);
            const char* sb = (const char*)S + (int64_t)rowbase * ngroups * 2;
            if constexpr (VS) {
                static_assert(U == 4, "four scales per load");
                t.sv[nt] = *(const uint2*)(sb + (int64_t)((k0 >> 7) + min(step_of(ks0, 0), steps - U)) * 2 + lo);
            } else {
#pragma unroll
                for (int u = 0; u < U; ++u)
                    t.s[nt][u] = *(const unsigned short*)(sb + (int64_t)((k0 + clamp_step(step_of(ks0, u)) * 128) / groupsize) * 2 + lo);
            }
        }
    };
    auto load_a = [&](ABatch& t, int ks0) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int j = 0; j < 4; ++j) t.a[u][mt][j] = *(const v4i*)(arow[mt] + clamp_step(step_of(ks0, u)) * 128 + 8 * j);
    };
    // k order of a dequantised word is [0,4,1,5,2,6,3,7]: bring the activation fragment into the same order
    auto perm_a = [&](ABatch& t) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const v4i x = t.a[u][mt][j];
                    v4i y;
                    y[0] = (int)__builtin_amdgcn_perm((unsigned)x[2], (unsigned)x[0], 0x05040100u);
                    y[1] = (int)__builtin_amdgcn_perm((unsigned)x[2], (unsigned)x[0], 0x07060302u);
                    y[2] = (int)__builtin_amdgcn_perm((unsigned)x[3], (unsigned)x[1], 0x05040100u);
                    y[3] = (int)__builtin_amdgcn_perm((unsigned)x[3], (unsigned)x[1], 0x07060302u);
                    t.a[u][mt][j] = y;
                }
    };
    auto mul = [&](const ABatch& ta, const BBatch& tb, int ks0, v4f (&acc)[NT][MT]) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const bool valid = step_of(ks0, u) < steps;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                unsigned short sraw;
                if constexpr (VS) sraw = (unsigned short)((u < 2 ? tb.sv[nt].x : tb.sv[nt].y) >> (16 * (u & 1)));
                else sraw = tb.s[nt][u];
                const float sc = valid ? f16_to_f32(sraw) : 0.f;
                v4f t[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) t[mt] = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const unsigned w = (unsigned)tb.w[nt][u][j], w8 = w >> 8;
                    const v8h bf = make8(deq_lo(w), deq_hi(w), deq_lo(w8), deq_hi(w8));
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        v8h a;
                        __builtin_memcpy(&a, &ta.a[u][mt][j], 16);
                        t[mt] = mfma_f16_16x16x32(a, bf, t[mt]);
                    }
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[nt][mt] += t[mt] * sc;
            }
        }
    };

    int tile = blockIdx.x;
    const int stride = gridDim.x;
    ABatch acur, anxt;
    BBatch bcur, bnxt, bnx2;
    // Every load of the ring is issued unconditionally (a tile index past the end is clamped to the last tile,
    // whose lines are then in cache): with loads under a condition the compiler cannot tell how many are in
    // flight and waits for all of them, the one just requested included, before it touches any.
    if (tile < ntiles) {
        // activations first (mostly L2 hits): they are permuted while the weights are still on their way
        load_a(acur, wave);
        load_b(bcur, tile, wave);
        if (RESIDENT) load_b(bnxt, min(tile + stride, ntiles - 1), wave);
        __builtin_amdgcn_sched_barrier(0);
        if (RESIDENT) perm_a(acur);
    }
    constexpr int NB = NT * MT;                          // 16x16 blocks per tile
    int parity = 0;
    v4f acc[NT][MT];
    auto clear_acc = [&]() {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (v4f){0.f, 0.f, 0.f, 0.f};
    };
    // cross-wave reduction of the K split, two alternating buffers: one barrier per tile
    auto finish = [&](int tl) __attribute__((always_inline)) {
        float* rbuf = red + parity * NW * NB * 256;
        parity ^= 1;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) *(v4f*)(rbuf + ((wave * NB + nt * MT + mt) * 64 + lane) * 4) = acc[nt][mt];
        __syncthreads();
        for (int o = threadIdx.x; o < NB * 256; o += NW * 64) {
            const int blk = o >> 8, nt = blk / MT, mt = blk - nt * MT, row16 = (o & 255) >> 4, col = o & 15;
            const int src = (blk * 64 + (row16 >> 2) * 16 + col) * 4 + (row16 & 3);
            const int m = m0 + 16 * mt + row16, n = (tl * NT + nt) * 16 + col;
            if (m >= M || n >= N) continue;
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) v += rbuf[w * NB * 256 + src];
            if (partial) partial[((int64_t)blockIdx.z * M + m) * N + n] = v;
            else C[(int64_t)m * N + n] = (_Float16)v;
        }
        clear_acc();
    };
    clear_acc();
    // The batches form a ring that is never copied (a register copy of a batch whose loads are in flight
    // would wait for them).
    if constexpr (RESIDENT) {
        auto one = [&](BBatch& cur, BBatch& fill) __attribute__((always_inline)) {
            load_b(fill, min(tile + 2 * stride, ntiles - 1), wave);
            mul(acur, cur, wave, acc);
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
        int ks0 = wave;
        auto one = [&](ABatch& ca, BBatch& cb, ABatch& fa, BBatch& fb) __attribute__((always_inline)) {
            const int nk = ks0 + NW * U;
            const bool more = step_of(nk, 0) < steps;
            const int nt = more ? tile : tile + stride;
            const bool any = nt < ntiles;
            const int fk = more ? nk : wave;
            if (any) { load_b(fb, nt, fk); load_a(fa, fk); }
            perm_a(ca);                                  // permuted when it becomes current, not while in flight
            mul(ca, cb, ks0, acc);
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

// Ring variant of the weight-streaming kernel for 128-wide groups, at most 16 rows per workgroup and a K range
// of at most 32 steps (steps % 4 == 0): wave w owns the four consecutive 128-K steps 4w .. 4w + 3 of every
// 16-column tile, its activation fragments stay in registers, and the packed words and group scales of the
// next DEPTH - 1 tiles are in flight in a ring of registers filled by hand-issued loads (see stream_ring.hpp:
// one s_waitcnt per tile that leaves exactly the younger tiles outstanding).
// BF: bf16 activations and outputs.  A nibble becomes the bf16 number 128 + q by OR-ing it into 0x4300 (exact:
// seven mantissa bits, q < 16), and the missing "- 136" of every product is the accumulator the MFMA chain of a
// step starts from: -136 * sum_k a[m][k] over the step, computed once per wave with the same MFMA and a weight
// fragment of constant 136 (the same for every tile).
template <int DEPTH, bool BF = false>
__global__ __launch_bounds__(512) void w4a16_nk_ring_kernel(
    const unsigned short* __restrict__ A, const int32_t* __restrict__ B, const _Float16* __restrict__ S,
    unsigned short* __restrict__ C, int M, int N, int Kfull, int Kc, float* __restrict__ partial) {
    using namespace llmk;
    constexpr int NW = 8, LPT = 5;                       // loads per tile and lane: four word vectors + the scales
    extern __shared__ float red[];                       // [2][NW][64][4]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int k0 = (int)blockIdx.z * Kc, K = min(Kc, Kfull - k0);
    const int steps = K >> 7, ngroups = Kfull >> 7, kwords = Kfull >> 3;
    const int m0 = blockIdx.y * 16;
    const int ntiles = (N + 15) >> 4;
    const bool wvalid = 4 * wave < steps;                // waves past the K range multiply by zero scales
    const int s0 = wvalid ? 4 * wave : 0;                // first step of this wave

    // ---- activations, requested first: row i of the wave's K slice (512 elements = 1 KiB) is one fully
    // coalesced load.  (Fetching the MFMA fragments straight from global memory costs 2 us per launch: every
    // 16-lane group of such a load touches 16 different cache lines, 16 bytes of each.)  They pass through a
    // wave-private LDS area once and stay in registers as fragments for every tile.
    v4i a[16];
    {
        // load 4 u + q: rows 4 q .. 4 q + 3 of the 256-byte slab of step u (a 16-lane group reads 256 contiguous bytes)
        const RingBase ab = ring_base((const char*)A + ((int64_t)k0 + s0 * 128) * 2);
        const uint32_t rowb = (uint32_t)(Kfull * 2), lrow = (uint32_t)(lane >> 4), lcol = 16u * (uint32_t)(lane & 15);
#define LLMK_LDA(u, q) a[4 * u + q] = ring_load_b128<u * 256>((uint32_t)min(m0 + 4 * q + (int)lrow, M - 1) * rowb + lcol, ab)
        LLMK_LDA(0, 0); LLMK_LDA(0, 1); LLMK_LDA(0, 2); LLMK_LDA(0, 3);
        LLMK_LDA(1, 0); LLMK_LDA(1, 1); LLMK_LDA(1, 2); LLMK_LDA(1, 3);
        LLMK_LDA(2, 0); LLMK_LDA(2, 1); LLMK_LDA(2, 2); LLMK_LDA(2, 3);
        LLMK_LDA(3, 0); LLMK_LDA(3, 1); LLMK_LDA(3, 2); LLMK_LDA(3, 3);
#undef LLMK_LDA
    }
    // ---- ring of weight tiles
    v4i w[DEPTH][4];
    v2i sv[DEPTH];
    const char* bb = (const char*)B + ((int64_t)(k0 >> 3) + s0 * 16) * 4;
    const char* sb = (const char*)S + ((int64_t)(k0 >> 7) + s0) * 2;
    auto issue = [&](v4i (&tw)[4], v2i& ts, int tile) __attribute__((always_inline)) {
        const int rowbase = tile * 16;
        const uint32_t row = (uint32_t)min(r, N - 1 - rowbase);             // rows past N repeat the last row
        const uint32_t vo = row * (uint32_t)(kwords * 4) + 16u * (uint32_t)g;
        const RingBase tb = ring_base(bb + (int64_t)rowbase * kwords * 4);
        tw[0] = ring_load_b128<0>(vo, tb);
        tw[1] = ring_load_b128<64>(vo, tb);
        tw[2] = ring_load_b128<128>(vo, tb);
        tw[3] = ring_load_b128<192>(vo, tb);
        ts = ring_load_b64<0>(row * (uint32_t)(ngroups * 2), ring_base(sb + (int64_t)rowbase * ngroups * 2));
    };
    int tile = blockIdx.x;
    const int stride = gridDim.x, last = ntiles - 1;
#pragma unroll
    for (int d = 0; d < DEPTH - 1; ++d) issue(w[d], sv[d], min(tile + d * stride, last));
    // the activations were requested before (DEPTH - 1) * LPT ring loads
    ring_wait16<(DEPTH - 1) * LPT>(a);
    {
        // one slab (16 rows x 256 bytes) at a time through the wave's LDS area; rows of 256 + 16 bytes, so that
        // the 16 rows of a fragment read fall into 16 different bank groups
        constexpr int AROW = 256 + 16;
        uint8_t* stage = (uint8_t*)red + 2 * NW * 256 * sizeof(float) + wave * (16 * AROW);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
#pragma unroll
            for (int q = 0; q < 4; ++q) *(v4i*)(stage + (4 * q + (lane >> 4)) * AROW + 16 * (lane & 15)) = a[4 * u + q];
            // fragment (u, j) of lane (r, g): elements 128 u + 32 g + 8 j .. + 7 of row r.  The k order of a
            // dequantised word is [0,4,1,5,2,6,3,7]: bring the activation fragment into the same order.
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const v4i x = *(const v4i*)(stage + r * AROW + 64 * g + 16 * j);
                v4i y;
                y[0] = (int)__builtin_amdgcn_perm((unsigned)x[2], (unsigned)x[0], 0x05040100u);
                y[1] = (int)__builtin_amdgcn_perm((unsigned)x[2], (unsigned)x[0], 0x07060302u);
                y[2] = (int)__builtin_amdgcn_perm((unsigned)x[3], (unsigned)x[1], 0x05040100u);
                y[3] = (int)__builtin_amdgcn_perm((unsigned)x[3], (unsigned)x[1], 0x07060302u);
                a[4 * u + j] = y;
            }
        }
    }

    // bf16: the bias of step u, -136 * sum_k a[row][k] in every column of the MFMA result
    v4f bias[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) bias[u] = (v4f){0.f, 0.f, 0.f, 0.f};
    if constexpr (BF) {
        const v4i c136 = {(int)0xc308c308u, (int)0xc308c308u, (int)0xc308c308u, (int)0xc308c308u};   // bf16 -136
        v8bf neg136;
        __builtin_memcpy(&neg136, &c136, 16);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v8bf af;
                __builtin_memcpy(&af, &a[4 * u + j], 16);
                bias[u] = mfma_bf16_16x16x32(af, neg136, bias[u]);
            }
    }

    int parity = 0;
    auto tile_done = [&](const v4i (&tw)[4], const v2i& ts, int tl) __attribute__((always_inline)) {
        v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const unsigned sraw = ((unsigned)(u < 2 ? ts[0] : ts[1]) >> (16 * (u & 1))) & 0xffffu;
            const float sc = wvalid ? f16_to_f32((unsigned short)sraw) : 0.f;
            v4f t = bias[u];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const unsigned x = (unsigned)tw[u][j];
                if constexpr (BF) {
                    // element pairs (k0,k4) (k1,k5) (k2,k6) (k3,k7) of the word, as for fp16
                    v4i bw;
                    bw[0] = (int)((x & 0x000f000fu) | 0x43004300u);
                    bw[1] = (int)(((x >> 4) & 0x000f000fu) | 0x43004300u);
                    bw[2] = (int)(((x >> 8) & 0x000f000fu) | 0x43004300u);
                    bw[3] = (int)(((x >> 12) & 0x000f000fu) | 0x43004300u);
                    v8bf bf, af;
                    __builtin_memcpy(&bf, &bw, 16);
                    __builtin_memcpy(&af, &a[4 * u + j], 16);
                    t = mfma_bf16_16x16x32(af, bf, t);
                } else {
                    const unsigned x8 = x >> 8;
                    const v8h bf = make8(deq_lo(x), deq_hi(x), deq_lo(x8), deq_hi(x8));
                    v8h af;
                    __builtin_memcpy(&af, &a[4 * u + j], 16);
                    t = mfma_f16_16x16x32(af, bf, t);
                }
            }
            acc += t * sc;
        }
        // cross-wave reduction of the K split, two alternating buffers: one barrier per tile
        float* rbuf = red + parity * NW * 256;
        parity ^= 1;
        *(v4f*)(rbuf + (wave * 64 + lane) * 4) = acc;
        __syncthreads();
        const int o = threadIdx.x;
        if (o < 256) {
            const int row16 = o >> 4, col = o & 15;
            const int src = ((row16 >> 2) * 16 + col) * 4 + (row16 & 3);
            const int m = m0 + row16, n = tl * 16 + col;
            float v = 0.f;
#pragma unroll
            for (int ww = 0; ww < NW; ++ww) v += rbuf[ww * 256 + src];
            if (m < M && n < N) {
                if (partial) partial[((int64_t)blockIdx.z * M + m) * N + n] = v;
                else C[(int64_t)m * N + n] = BF ? f32_to_bf16(v) : f32_to_f16(v);
            }
        }
    };
    // (the loop is left behind a full wait: no path of the flow graph may lead from a request back to the loop
    // head without passing a wait that covers it, and the clamped requests of the last tiles are drained)
    // Whole rounds of DEPTH tiles run in a loop whose body has no branch (every request and every wait is
    // executed on every path, so what the static check of the assembly sees is what runs); the last
    // my_tiles % DEPTH tiles, all requested by then, follow as straight-line code.  Requests past the last tile
    // of the workgroup are clamped to the last tile of the matrix (cache hits) and never consumed.
    const int my_tiles = (ntiles - (int)blockIdx.x + stride - 1) / stride;
    auto slot = [&](auto dc) __attribute__((always_inline)) {
        constexpr int d = decltype(dc)::value, NEXT = DEPTH - 1;
        issue(w[(d + NEXT) % DEPTH], sv[(d + NEXT) % DEPTH], min(tile + NEXT * stride, last));
        ring_wait<(DEPTH - 1) * LPT>(w[d][0], w[d][1], w[d][2], w[d][3], sv[d]);
        tile_done(w[d], sv[d], tile);
        tile += stride;
    };
    auto tail = [&](auto dc) __attribute__((always_inline)) {
        constexpr int d = decltype(dc)::value;
        ring_wait<(DEPTH - 2 - d) * LPT>(w[d][0], w[d][1], w[d][2], w[d][3], sv[d]);
        tile_done(w[d], sv[d], tile);
        tile += stride;
    };
    static_assert(DEPTH >= 2 && DEPTH <= 4, "ring slots are spelled out below");
    for (int rd = my_tiles / DEPTH; rd > 0; --rd) {
        slot(std::integral_constant<int, 0>{});
        if constexpr (DEPTH > 1) slot(std::integral_constant<int, 1>{});
        if constexpr (DEPTH > 2) slot(std::integral_constant<int, 2>{});
        if constexpr (DEPTH > 3) slot(std::integral_constant<int, 3>{});
    }
    const int rem = my_tiles % DEPTH;
    if constexpr (DEPTH > 1) { if (rem > 0) tail(std::integral_constant<int, 0>{}); }
    if constexpr (DEPTH > 2) { if (rem > 1) tail(std::integral_constant<int, 1>{}); }
    if constexpr (DEPTH > 3) { if (rem > 2) tail(std::integral_constant<int, 2>{}); }
    ring_drain<0>();
}

// The ring kernel takes 128-wide groups, K ranges of at most 32 steps in whole four-step shares, 8-byte aligned
// scale rows and operands below 4 GiB (32-bit lane offsets); nz = number of K ranges.
bool nk_ring_ok(int64_t M, int64_t N, int64_t K, int groupsize, int nz, const void* S) {
    const int64_t steps_all = K >> 7, steps = (steps_all + nz - 1) / nz;
    return groupsize == 128 && steps <= 32 && steps_all % 4 == 0 && steps % 4 == 0 && !(((uintptr_t)S) & 7) &&
           N * (K / 2) < (1ll << 32) && M * K * 2 < (1ll << 32);
}

// fp16 or bf16 (bf) activations / outputs; partial: fp32 planes for nz > 1 (a summing pass follows)
int launch_nk_ring(const void* A, const int32_t* B, const _Float16* S, void* C, int M, int N, int K, int nz, float* partial,
                   bool bf, hipStream_t st) {
    const int steps_all = K >> 7, steps = (steps_all + nz - 1) / nz, Kc = steps * 128;
    const int ntiles = (N + 15) / 16, mtiles = (M + 15) / 16, rows = mtiles * nz;
    // One workgroup per CU and row tile, ring depth = tiles per workgroup (two to four).  Two workgroups per CU
    // with rings of two measured slower (20.4 vs 18.2 us at N = 28672): every workgroup reads all the activations
    // of its row tile, and that traffic doubles.
    const int cus = std::max(1, llmk_device_cus() > 0 ? llmk_device_cus() : LLMK_CUS);
    const int wg = min(ntiles, max(1, cus / min(rows, cus)));
    const int per_wg = (ntiles + wg - 1) / wg;
    dim3 rgrid((unsigned)((ntiles + per_wg - 1) / per_wg), (unsigned)mtiles, (unsigned)nz);
    // reduction buffers + the wave-private staging area of the activations
    const size_t rsmem = 2 * 8 * 256 * sizeof(float) + 8 * 16 * (256 + 16);
    const unsigned short* a16 = (const unsigned short*)A;
    unsigned short* c16 = (unsigned short*)C;
    float* part = nz > 1 ? partial : nullptr;
#define LLMK_RING(D)                                                                                             \
    do {                                                                                                         \
        if (bf) w4a16_nk_ring_kernel<D, true><<<rgrid, 512, rsmem, st>>>(a16, B, S, c16, M, N, K, Kc, part);      \
        else w4a16_nk_ring_kernel<D, false><<<rgrid, 512, rsmem, st>>>(a16, B, S, c16, M, N, K, Kc, part);        \
    } while (0)
    if (per_wg >= 4) LLMK_RING(4);
    else if (per_wg == 3) LLMK_RING(3);
    else LLMK_RING(2);
#undef LLMK_RING
    LLMK_CHECK_LAUNCH("gemm_w4a16_nk(ring)");
    if (nz > 1) {
        const int64_t mn = (int64_t)M * N;
        if (bf) llmk::splitk_sum_kernel<LLMK_BF16><<<(unsigned)cdiv64(cdiv64(mn, 4), 256), 256, 0, st>>>(partial, C, mn, nz);
        else splitk_reduce_f16_kernel<<<(unsigned)cdiv64(mn, 4 * 256), 256, 0, st>>>(partial, (_Float16*)C, mn, nz);
        LLMK_CHECK_LAUNCH("gemm_w4a16_nk(reduce)");
    }
    return LLMK_OK;
}

template <int MT, int NT>
int launch_nk_stream(const _Float16* A, const int32_t* B, const _Float16* S, _Float16* C, int M, int N, int K, int groupsize,
                     int nz, float* partial, hipStream_t st) {
    if constexpr (MT == 1 && NT == 1) {
        if (nk_ring_ok(M, N, K, groupsize, nz, S)) return launch_nk_ring(A, B, S, C, M, N, K, nz, partial, false, st);
    }
    constexpr int U = MT == 1 ? 4 : (MT == 2 ? 2 : 1);
    // nz K ranges, equally long up to one step
    const int steps_all = K >> 7, steps = (steps_all + nz - 1) / nz, Kc = steps * 128;
    const int ntiles = (N + 16 * NT - 1) / (16 * NT), mtiles = (M + 16 * MT - 1) / (16 * MT);
    const bool resident = steps <= 8 * U;
    const size_t smem = (size_t)2 * 8 * NT * MT * 256 * sizeof(float);
    static std::atomic<int> slots_cache[2];
    int slots[2] = {slots_cache[0].load(std::memory_order_relaxed), slots_cache[1].load(std::memory_order_relaxed)};
    if (slots[resident] == 0) {
        int dev = 0, cus = 0, per_cu = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (e == hipSuccess)
            e = resident ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, w4a16_nk_stream_kernel<MT, NT, true>, 512, smem)
                         : hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, w4a16_nk_stream_kernel<MT, NT, false>, 512, smem);
        if (e != hipSuccess) LLMK_FAIL(LLMK_ERR_LAUNCH, "gemm_w4a16_nk: occupancy query failed: %s", hipGetErrorString(e));
        slots[resident] = max(1, cus * max(1, per_cu));
        slots_cache[resident].store(slots[resident], std::memory_order_relaxed);
    }
    const int rows = mtiles * nz;
    int gx = min(ntiles, max(1, slots[resident] / min(rows, slots[resident])));
    { const int per_wg = (ntiles + gx - 1) / gx; gx = (ntiles + per_wg - 1) / per_wg; }   // equal tile counts
    dim3 grid((unsigned)gx, (unsigned)mtiles, (unsigned)nz);
    float* part = nz > 1 ? partial : nullptr;
    bool launched = false;
    if constexpr (U == 4) {
        // consecutive steps per wave and one load for their four scales
        if (!launched && groupsize == 128 && steps_all % 4 == 0 && steps % 4 == 0 && !(((uintptr_t)S) & 7)) {
            if (resident) w4a16_nk_stream_kernel<MT, NT, true, true><<<grid, 512, smem, st>>>(A, B, S, C, M, N, K, groupsize, Kc, part);
            else w4a16_nk_stream_kernel<MT, NT, false, true><<<grid, 512, smem, st>>>(A, B, S, C, M, N, K, groupsize, Kc, part);
            launched = true;
        }
    }
    if (!launched) {
        if (resident) w4a16_nk_stream_kernel<MT, NT, true><<<grid, 512, smem, st>>>(A, B, S, C, M, N, K, groupsize, Kc, part);
        else w4a16_nk_stream_kernel<MT, NT, false><<<grid, 512, smem, st>>>(A, B, S, C, M, N, K, groupsize, Kc, part);
    }
    LLMK_CHECK_LAUNCH("gemm_w4a16_nk(stream)");
    if (nz > 1) {
        splitk_reduce_f16_kernel<<<(unsigned)cdiv64((int64_t)M * N, 4 * 256), 256, 0, st>>>(partial, C, (int64_t)M * N, nz);
        LLMK_CHECK_LAUNCH("gemm_w4a16_nk(reduce)");
    }
    return LLMK_OK;
}

// Rows for which the 128-column tile kernels expand the 4-bit weights themselves: 65 to 512 always (measured
// 1.3-2.8x faster than the separate expansion pass up to 256 rows, even to 1.4x at 512); 33 to 64 when the
// weight matrix is large, where the tile kernel with split-K beats the weight-streaming kernels (which read
// the activations once per 16 columns), provided the scratch for its partial sums is there.
// `wide`: the layout also has the expansion inside the 256-column tile kernel (row-packed layout only).  Up to 512
// rows the fused tile kernels win everywhere (1.3-2.8x); beyond that the fused 256 x 256 kernel wins over the
// dequantisation pass + fp16 GEMM only when the problem takes two or more rounds of 256 tiles (4096 x 28672 x 4096:
// 741 vs 758 us, 2048 x 14336 x 4096: 198 vs 201 us), and loses on one round (4096^3: 109 vs 105 us).
bool w4_tiles_expand(int64_t M, int64_t N, int64_t K, const void* workspace, int64_t workspace_bytes, bool wide = false) {
    if (M > 512) return wide && ((M + 255) / 256) * ((N + 255) / 256) >= 512;
    if (M > 64) return true;
    if (M <= 32 || K % 64) return false;
    const int64_t nk = N * K;
    if (!(K > 4096 ? nk >= ((int64_t)32 << 20) : nk >= ((int64_t)96 << 20))) return false;
    const int z = llmk::splitk_factor_half(M, N, K);
    return z <= 1 || (workspace && workspace_bytes >= (int64_t)z * M * N * 4 && !((uintptr_t)workspace & 15));
}

// launch shape of the Marlin-layout kernel for a given problem
struct MarlinPlan {
    int mt, nw, mblocks, col_groups, z, steps_per_z;
};

MarlinPlan marlin_plan(int64_t M, int64_t N, int64_t K) {
    MarlinPlan pl{};
    pl.mt = 1;                                              // 16-row workgroups side by side (measured faster than taller ones)
    pl.nw = 8;                                              // nw * mt * 8 KiB of reduction LDS <= 64 KiB
    pl.mblocks = (int)cdiv64(M, 16 * pl.mt);
    pl.col_groups = (int)((N / 64 + 1) / 2);
    const int total_steps = (int)((K / 16 + 1) / 2);
    // split K over workgroups until the grid covers the chip; every slice keeps >= nw steps
    int z = 1;
    if (M <= 64)
        while ((int64_t)pl.col_groups * pl.mblocks * z < 256 && total_steps / (z * 2) >= pl.nw) z *= 2;
    pl.z = z;
    pl.steps_per_z = (total_steps + z - 1) / z;
    return pl;
}

}  // namespace

extern "C" int64_t llmk_gemm_w4a16_marlin_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    if (M > 64) {                                        // dequantised fp16 copy of W for the tiled GEMM (+ split-K partials)
        if (K % 64) return 0;
        const int z = llmk::splitk_factor_half(M, N, K);
        return ((N * K * 2 + 255) & ~(int64_t)255) + (z > 1 ? (int64_t)z * M * N * 4 : 0);
    }
    const MarlinPlan pl = marlin_plan(M, N, K);
    const int64_t zt = M > 16 && K % 64 == 0 ? llmk::splitk_factor_half(M, N, K) : 1;   // tile kernels with split-K
    const int64_t z = pl.z > zt ? pl.z : zt;
    return z > 1 ? z * M * N * 4 : 0;
}

extern "C" int llmk_gemm_w4a16_marlin(const void* a, const int32_t* b, void* c, const void* s, int64_t M, int64_t N,
                                      int64_t K, int groupsize, void* workspace, int64_t workspace_bytes,
                                      void* stream) {
    // the reference launcher returns -1 for any dimension not divisible by 16 (marlin_w4a16_gemm.cu:300-302)
    if (M % 16 || N % 16 || K % 16 || M < 0 || N < 0 || K < 0)
        LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a16_marlin: M, N, K must be multiples of 16 (M=%lld N=%lld K=%lld)", (long long)M, (long long)N, (long long)K);
    if (N % 64) LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a16_marlin: N=%lld must be a multiple of 64 (packed chunk width)", (long long)N);
    if (M == 0 || N == 0) return LLMK_OK;
    if (K == 0) LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a16_marlin: K == 0");
    if (groupsize == -1) groupsize = (int)K;
    if (groupsize < 16 || groupsize % 16 || K % groupsize)
        LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a16_marlin: groupsize=%d must be a multiple of 16 dividing K=%lld", groupsize, (long long)K);
    if (!a || !b || !c || !s) LLMK_FAIL(LLMK_ERR_ARG, "gemm_w4a16_marlin: null pointer");
    if (((uintptr_t)a | (uintptr_t)b | (uintptr_t)s) & 15) LLMK_FAIL(LLMK_ERR_ARG, "gemm_w4a16_marlin: operands must be 16-byte aligned");
    if (M > 0x7fffffff / 2 || N > 0x7fffffff / 2 || K > 0x7fffffff / 2) LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a16_marlin: dimension too large");

    hipStream_t st = (hipStream_t)stream;
    if (w4_tiles_expand(M, N, K, workspace, workspace_bytes) && K % 64 == 0 && groupsize % 64 == 0) {
        // mid-size M: the 128-column tile kernels expand the Marlin units themselves (see gemm_w4a16_nk)
        llmk::DirectArgs p{};
        p.a = (const uint8_t*)a; p.b = (const uint8_t*)b; p.b_s = s; p.c = c; p.c_dtype = LLMK_F16;
        p.M = (int)M; p.N = (int)N; p.K = (int)K; p.E = 1; p.group = groupsize;
        if (llmk::dma_eligible(p, 2))
            return llmk::launch_big_half<llmk::K_W4MARLIN, false>(p, st, "gemm_w4a16_marlin(fused tiles)", workspace, workspace_bytes);
    }
    if (M > 64 && K % 64 == 0 && workspace && workspace_bytes >= N * K * 2 && !((uintptr_t)workspace & 15)) {
        // compute-bound: expand W once to fp16 [N, K], then run the tiled MFMA GEMM on it
        llmk::DirectArgs p{};
        p.a = (const uint8_t*)a; p.b = (const uint8_t*)workspace; p.c = c; p.c_dtype = LLMK_F16;
        p.M = (int)M; p.N = (int)N; p.K = (int)K; p.E = 1;
        if (llmk::dma_eligible(p, 2)) {
            dim3 dgrid((unsigned)(N / 64), (unsigned)cdiv64(K, 128));
            marlin_dequant_kernel<<<dgrid, 256, 0, st>>>((const v4i*)b, (const _Float16*)s, (_Float16*)workspace, (int)N, (int)K, groupsize);
            LLMK_CHECK_LAUNCH("gemm_w4a16_marlin(dequant)");
            const int64_t used = (N * K * 2 + 255) & ~(int64_t)255;
            return llmk::launch_big_half<llmk::K_F16, false>(p, st, "gemm_w4a16_marlin(tiled)", (uint8_t*)workspace + used,
                                                             workspace_bytes > used ? workspace_bytes - used : 0);
        }
    }
    MarlinPlan pl = marlin_plan(M, N, K);
    if (pl.z > 1 && (!workspace || workspace_bytes < (int64_t)pl.z * M * N * 4 || (((uintptr_t)workspace) & 15) || (((uintptr_t)c) & 7))) {
        pl.z = 1;                                   // no scratch: every workgroup walks all of K
        pl.steps_per_z = (int)((K / 16 + 1) / 2);
    }
    const _Float16* A = (const _Float16*)a;
    const v4i* B = (const v4i*)b;
    const _Float16* S = (const _Float16*)s;
    _Float16* C = (_Float16*)c;
    float* ws = (float*)workspace;
    dim3 grid(pl.col_groups, pl.mblocks, pl.z), blk(pl.nw * 64);
    const size_t red_bytes = (size_t)pl.nw * pl.mt * 32 * 64 * sizeof(float);
    const size_t a_bytes = (size_t)16 * pl.mt * ((size_t)pl.steps_per_z * 64 + 16);     // activation image of one K range
    // staged while every workgroup fits on the chip at once; with several rounds of workgroups the unoverlapped
    // staging of each costs more than the global fragment loads (measured at N = 128256: 88 vs 84 us)
    const bool a_lds = a_bytes <= 144 * 1024 && (int64_t)pl.col_groups * pl.mblocks * pl.z <= 512;
    const size_t smem = a_lds && a_bytes > red_bytes ? a_bytes : red_bytes;
    if (smem > 64 * 1024) {
        static std::atomic<uint64_t> cfg_a{0}, cfg_b{0};
        if (int rc = llmk_reserve_lds((const void*)w4a16_marlin_kernel<1, 8, true, true>, 160 * 1024, cfg_a, "gemm_w4a16_marlin")) return rc;
        if (int rc = llmk_reserve_lds((const void*)w4a16_marlin_kernel<1, 8, false, true>, 160 * 1024, cfg_b, "gemm_w4a16_marlin")) return rc;
    }
#define LLMK_MARLIN_LAUNCH(MT, NW)                                                                              \
    do {                                                                                                        \
        if (pl.z > 1 && a_lds) w4a16_marlin_kernel<MT, NW, true, true><<<grid, blk, smem, st>>>(A, B, S, C, ws, (int)M, (int)N, (int)K, groupsize, pl.steps_per_z); \
        else if (pl.z > 1) w4a16_marlin_kernel<MT, NW, true><<<grid, blk, smem, st>>>(A, B, S, C, ws, (int)M, (int)N, (int)K, groupsize, pl.steps_per_z); \
        else if (a_lds) w4a16_marlin_kernel<MT, NW, false, true><<<grid, blk, smem, st>>>(A, B, S, C, nullptr, (int)M, (int)N, (int)K, groupsize, pl.steps_per_z); \
        else w4a16_marlin_kernel<MT, NW, false><<<grid, blk, smem, st>>>(A, B, S, C, nullptr, (int)M, (int)N, (int)K, groupsize, pl.steps_per_z); \
    } while (0)
    LLMK_MARLIN_LAUNCH(1, 8);
#undef LLMK_MARLIN_LAUNCH
    LLMK_CHECK_LAUNCH("gemm_w4a16_marlin");
    if (pl.z > 1) {
        splitk_reduce_f16_kernel<<<(unsigned)cdiv64(M * N, 4 * 256), 256, 0, st>>>((const float*)workspace, C, M * N, pl.z);
        LLMK_CHECK_LAUNCH("gemm_w4a16_marlin(reduce)");
    }
    return LLMK_OK;
}

extern "C" int llmk_gemm_w4a16_nk(const void* a, const int32_t* b_packed, void* c, const void* s, int ac_dtype,
                                  int64_t M, int64_t N, int64_t K, int groupsize, void* workspace,
                                  int64_t workspace_bytes, void* stream) {
    if (ac_dtype != LLMK_F16 && ac_dtype != LLMK_BF16) LLMK_FAIL(LLMK_ERR_DTYPE, "gemm_w4a16_nk: activations / outputs must be fp16 or bf16 (dtype code %d)", ac_dtype);
    const bool bf = ac_dtype == LLMK_BF16;
    if (M < 0 || N < 0 || K < 0 || K % 128) LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a16_nk: K=%lld must be a multiple of 128", (long long)K);
    if (M == 0 || N == 0) return LLMK_OK;
    if (K == 0) LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a16_nk: K == 0");
    if (groupsize == -1) groupsize = (int)K;
    if (groupsize < 8 || groupsize % 8 || K % groupsize)
        LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a16_nk: groupsize=%d must be a multiple of 8 dividing K", groupsize);
    if (!a || !b_packed || !c || !s) LLMK_FAIL(LLMK_ERR_ARG, "gemm_w4a16_nk: null pointer");
    if (((uintptr_t)a | (uintptr_t)b_packed) & 15) LLMK_FAIL(LLMK_ERR_ARG, "gemm_w4a16_nk: operands must be 16-byte aligned");
    if (M > 0x7fffffff / 2 || N > 0x7fffffff / 2 || K > 0x7fffffff / 2) LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a16_nk: dimension too large");
    hipStream_t st = (hipStream_t)stream;
    const _Float16* A = (const _Float16*)a;
    const _Float16* S = (const _Float16*)s;
    _Float16* C = (_Float16*)c;
    // bf16: the weight-streaming ring kernel for decode sizes, everything else through the bf16 copy of W
    const int nz_bf = (int)((K / 128 + 31) / 32);
    const bool bf_ring = bf && M <= 64 && nk_ring_ok(M, N, K, groupsize, nz_bf, s) && !((uintptr_t)c & 7) &&
                         (nz_bf == 1 || ((M * N) % 4 == 0 && workspace && workspace_bytes >= (int64_t)nz_bf * M * N * 4 &&
                                         !((uintptr_t)workspace & 15)));
    if (bf_ring) return launch_nk_ring(a, b_packed, S, c, (int)M, (int)N, (int)K, nz_bf, (float*)workspace, true, st);
    if (!bf && w4_tiles_expand(M, N, K, workspace, workspace_bytes, true) && K % 64 == 0 && groupsize % 64 == 0) {
        // mid-size M: the 128-column tile kernels expand the packed words themselves (every weight byte is
        // read once; the separate expansion pass would write and re-read four times as much).
        llmk::DirectArgs p{};
        p.a = (const uint8_t*)a; p.b = (const uint8_t*)b_packed; p.b_s = s; p.c = c; p.c_dtype = LLMK_F16;
        p.M = (int)M; p.N = (int)N; p.K = (int)K; p.E = 1; p.group = groupsize;
        // few column tiles and short rows: the 64-column kernel with 512-byte K steps (128 x 4096 x 4096: 18.3 -> 14 us)
        if (2 * K <= 8192 && llmk::mid_wanted(M, N, 2 * K)) {       // (rows beyond 8 KB: measured only for the 8-bit kinds)
            llmk::MidPlan pl = llmk::mid_plan(M, N, 2 * K);
            if (pl.z > 1 && !(workspace && workspace_bytes >= (int64_t)pl.z * M * N * 4 && !((uintptr_t)workspace & 15))) pl.z = 1;
            if (llmk::mid_eligible<llmk::K_W4NK>(p, pl.mt, pl.z)) {
                if (pl.z > 1) { p.partial = (float*)workspace; p.ksplit = pl.z; }
                return pl.mt == 4 ? llmk::launch_mid<llmk::K_W4NK, 4>(p, st, "gemm_w4a16_nk(mid)")
                                  : llmk::launch_mid<llmk::K_W4NK, 2>(p, st, "gemm_w4a16_nk(mid)");
            }
        }
        // wider weights on one round of 128-column tiles: the 128-column form of that kernel
        if (2 * K <= 8192 && llmk::midw_wanted(M, N, 2 * K) && llmk::dma_eligible(p, 2) && (groupsize & (groupsize - 1)) == 0) {       // (longer rows: measured for fp8 only)
            llmk::MidPlan pl = llmk::midw_plan(M, N, 2 * K);
            if (pl.z > 1 && !(workspace && workspace_bytes >= (int64_t)pl.z * M * N * 4 && !((uintptr_t)workspace & 15))) pl.z = 1;
            if (pl.z > 1) { p.partial = (float*)workspace; p.ksplit = pl.z; }
            return pl.mt == 4 ? llmk::launch_mid<llmk::K_W4NK, 4, false, true>(p, st, "gemm_w4a16_nk(mid, 128 columns)")
                              : llmk::launch_mid<llmk::K_W4NK, 8, false, true>(p, st, "gemm_w4a16_nk(mid, 128 columns)");
        }
        if (llmk::dma_eligible(p, 2))
            return llmk::launch_big_half<llmk::K_W4NK, false>(p, st, "gemm_w4a16_nk(fused tiles)", workspace, workspace_bytes);
    }
    if ((M > 64 || bf) && K % 64 == 0 && workspace && workspace_bytes >= N * K * 2 && !((uintptr_t)workspace & 15)) {
        // compute-bound: expand W once to fp16 / bf16 [N, K], then run the tiled MFMA GEMM on it
        llmk::DirectArgs p{};
        p.a = (const uint8_t*)a; p.b = (const uint8_t*)workspace; p.c = c; p.c_dtype = ac_dtype;
        p.M = (int)M; p.N = (int)N; p.K = (int)K; p.E = 1;
        if (llmk::dma_eligible(p, 2)) {
            const unsigned blocks = (unsigned)cdiv64(N * (K / 8), 256);
            if (bf) nk_dequant_bf16_kernel<<<blocks, 256, 0, st>>>(b_packed, S, (unsigned short*)workspace, N, K, groupsize);
            else nk_dequant_kernel<<<blocks, 256, 0, st>>>(b_packed, S, (_Float16*)workspace, N, K, groupsize);
            LLMK_CHECK_LAUNCH("gemm_w4a16_nk(dequant)");
            const int64_t used = (N * K * 2 + 255) & ~(int64_t)255;
            void* rest = (uint8_t*)workspace + used;
            const int64_t rest_bytes = workspace_bytes > used ? workspace_bytes - used : 0;
            if (bf) return llmk::launch_big_half<llmk::K_BF16, false>(p, st, "gemm_w4a16_nk(tiled, bf16)", rest, rest_bytes);
            return llmk::launch_big_half<llmk::K_F16, false>(p, st, "gemm_w4a16_nk(tiled)", rest, rest_bytes);
        }
    }
    if (bf) LLMK_FAIL(LLMK_ERR_ARG, "gemm_w4a16_nk: this bf16 call needs a 16-byte aligned workspace of N*K*2 = %lld bytes (bf16 copy of W)",
                      (long long)(N * K * 2));
    if (groupsize % 128 == 0 && M <= 64) {
        // one 16-column block per tile: two blocks per tile (NT = 2) measured slower at every shape tried.
        // While the activations of a 16-row workgroup stay resident (K <= 4096), such workgroups side by side
        // beat taller ones by up to 2x.
        // K > 4096: ranges of at most 4096 (each with resident activations) and fp32 partial sums, when the
        // workspace holds them
        const int nz = (int)((K / 128 + 31) / 32);
        const bool ranges = nz > 1 && (M * N) % 4 == 0 && K % groupsize == 0 && ((K / 128 + nz - 1) / nz * 128) % groupsize == 0 &&
                            workspace && workspace_bytes >= (int64_t)nz * M * N * 4 && !((uintptr_t)workspace & 15) && !((uintptr_t)c & 7);
        if (ranges) return launch_nk_stream<1, 1>(A, b_packed, S, C, (int)M, (int)N, (int)K, groupsize, nz, (float*)workspace, st);
        if (M <= 16 || K <= 4096) return launch_nk_stream<1, 1>(A, b_packed, S, C, (int)M, (int)N, (int)K, groupsize, 1, nullptr, st);
        if (M <= 32) return launch_nk_stream<2, 1>(A, b_packed, S, C, (int)M, (int)N, (int)K, groupsize, 1, nullptr, st);
        return launch_nk_stream<4, 1>(A, b_packed, S, C, (int)M, (int)N, (int)K, groupsize, 1, nullptr, st);
    }
    const unsigned gx = (unsigned)cdiv64(N, 16);
    if (M <= 16) {
        constexpr int NW = 8;
        w4a16_nk_kernel<1, NW><<<dim3(gx, 1), NW * 64, (NW / 2) * 4 * 64 * sizeof(float), st>>>(A, b_packed, S, C, (int)M, (int)N, (int)K, groupsize);
    } else {
        constexpr int MT = 4, NW = 4;
        w4a16_nk_kernel<MT, NW><<<dim3(gx, (unsigned)cdiv64(M, 16 * MT)), NW * 64, (NW / 2) * MT * 4 * 64 * sizeof(float), st>>>(A, b_packed, S, C, (int)M, (int)N, (int)K, groupsize);
    }
    LLMK_CHECK_LAUNCH("gemm_w4a16_nk");
    return LLMK_OK;
}
