// W4A8 GEMM: int8 activations x row-packed uint4 weights with two-level scales.
#include "gemm_wide.hpp"
#include "stream_ring.hpp"

using namespace llmk;

namespace {

// 16-bit block scales that the same launch widens to fp32 for the int8 GEMM behind it (blocks past the expansion's):
// saves that GEMM a launch of its own for the activation scales
struct W4A8Widen {
    const void* a_s; const void* b_s;
    float* a_s32; float* b_s32;
    int64_t n_a, n_b;
    int s_dtype;
    unsigned first_block;       // 0: nothing to widen
};

// packed [N/8, K] int32 -> b8 [N, K] int8 with b8 = int8(int8(q - z4) * s4) (two's-complement wrap)
__global__ void w4a8_expand_kernel(const int32_t* __restrict__ packed, const int8_t* __restrict__ s4,
                                   const int8_t* __restrict__ z4, int8_t* __restrict__ out,
                                   int64_t N, int64_t K, int group, W4A8Widen wd) {
    if (wd.first_block && blockIdx.x >= wd.first_block) {
        const int64_t i = (int64_t)(blockIdx.x - wd.first_block) * blockDim.x + threadIdx.x;
        if (i < wd.n_a) wd.a_s32[i] = ld_scale(wd.a_s, i, wd.s_dtype);
        else if (i < wd.n_a + wd.n_b) wd.b_s32[i - wd.n_a] = ld_scale(wd.b_s, i - wd.n_a, wd.s_dtype);
        return;
    }
    // one thread: 8 rows x 4 consecutive k
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t kq = K / 4;
    if (idx >= (N / 8) * kq) return;
    const int64_t pr = idx / kq, k = (idx - pr * kq) * 4;
    const v4i w = *(const v4i*)(packed + pr * K + k);
    const int64_t kg = K / group;
    const int64_t gi = k / group;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int64_t n = pr * 8 + i;
        const int z = z4[n * kg + gi], s = s4[n * kg + gi];
        unsigned o = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int q = (w[j] >> (4 * i)) & 0xf;
            const int d = (int)(int8_t)(q - z);
            o |= ((unsigned)((d * s) & 0xff)) << (8 * j);
        }
        *(unsigned*)(out + n * K + k) = o;
    }
}


// ------------------------------------------------------------------------------------------------------------
// Fused decode-size kernel (small M, 128-wide second-level groups, K in ranges of at most 4096 per workgroup).  The packed words are streamed
// HBM -> registers -> LDS fully coalesced; each lane then picks the nibble of its column out of the words it
// needs, and the dequantisation (q - z4) * s4 is moved out of the inner product:
//     sum_k a_k (q_k - z) s = s (sum_k a_k q_k - z sum_k a_k)      per 128-K group,
// exact whenever (q - z) s fits int8 for q in 0..15 (weight_quant's output nearly always does).  A wave whose
// lanes hold out-of-range (z4, s4) for a step dequantises that step nibble by nibble with the int8 wrap.
//
// Workgroup = 8 waves on 16 MT rows x 16 columns (two packed rows), persistent over column tiles; each wave
// takes a run of consecutive 128-K steps; activation fragments, their per-group sums and scales stay resident.  The
// loads of tiles i+1 and i+2 are in flight while tile i is multiplied: a ring of three register sets filled by
// hand-issued loads and released by one hand-counted wait per tile (stream_ring.hpp; with ordinary loads the
// compiler ended every conditional request of the loop with a full wait).  Past the last tile the same number of
// loads is still issued (all lanes on one hot line) so that the wait counts stay exact.
struct W4A8Args {
    const int8_t* a; const void* a_s; const int32_t* packed; const void* b_s; const int8_t* s4; const int8_t* z4;
    void* c; int c_dtype; int M, N, K;
    int Kc;             // K range of one workgroup (multiple of 128, at most 4096); gridDim.z ranges cover K
    float* partial;     // more than one range: fp32 partial sums [gridDim.z][M][N], summed by a second kernel
};

template <int MT, int SDT, int ROUNDS>
__global__ __launch_bounds__(512) void w4a8_stream_kernel(W4A8Args p) {
    constexpr int NW = 8, U = 4, D = 3;
    constexpr bool TAB_REGS = MT == 1;                    // per-row sums and scales in registers, else in LDS
    constexpr int ROWSTRIDE = ROUNDS * 8192 + 64;         // +64: the two packed rows of a tile start in different banks
    constexpr int TB = 2 * ROWSTRIDE;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4, col8 = r & 7, half = r >> 3;
    // this workgroup's K range: elements [k0, k0 + K) of rows that are Kfull long
    const int M = p.M, N = p.N, Kfull = p.K, sfull = Kfull >> 7;
    const int k0 = (int)blockIdx.z * p.Kc, sk0 = k0 >> 7;
    const int K = min(p.Kc, Kfull - k0), steps = K >> 7;
    const int m0 = blockIdx.y * 16 * MT;
    const int ntiles = (N + 15) >> 4, np = N >> 3;
    // wave w multiplies the `cs` consecutive 128-K steps from w * cs: its zero points and second-level scales
    // of a column are then the bytes of one dword
    const int cs = (steps + NW - 1) / NW, ks0 = wave * cs;
    auto step_ok = [&](int u) { return u < cs && ks0 + u < steps; };

    float* red = (float*)smem;                            // [2][NW][MT][256]
    float2* tab = (float2*)(red + 2 * NW * MT * 256);     // [MT*16][steps]: {activation scale, activation byte sum}
    uint8_t* tbuf = (uint8_t*)(tab + MT * 16 * steps);    // two staged tiles

    // z / s: the four zero points and second-level scales of this lane's column, one byte per step of the wave;
    // bs: the block scale of step (lane & 3)
    struct TileRegs { int z, s, bs; v4i w[2 * ROUNDS]; };
    constexpr int LPT = 2 * ROUNDS + 3;                   // loads per tile and lane
    const RingBase zbase = ring_base(p.z4), sbase = ring_base(p.s4), bsbase = ring_base(p.b_s);
    auto issue_tile = [&](TileRegs& t, int tile) __attribute__((always_inline)) {
        const bool live = tile < ntiles;
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
            const int prow = live ? min(tile * 2 + hh, np - 1) : 0;
            const RingBase rowp = ring_base((const uint8_t*)p.packed + ((int64_t)prow * Kfull + k0) * 4);
#pragma unroll
            for (int rd = 0; rd < ROUNDS; ++rd) {
                const uint32_t off = (uint32_t)(rd * 8192 + wave * 1024 + lane * 16);
                t.w[hh * ROUNDS + rd] = ring_load_b128<0>(live ? min(off, (uint32_t)(K * 4 - 16)) : 0u, rowp);
            }
        }
        const int n = live ? min(tile * 16 + r, N - 1) : 0;
        // dword at byte n * (K / 128) + first step of this wave, pulled back inside the table at its very end (the
        // shift that undoes the pull is applied where the bytes are used)
        const int64_t want = (int64_t)n * sfull + sk0 + ks0, last = (int64_t)N * sfull - 4;
        const uint32_t at = (uint32_t)min(want, last);
        t.z = ring_load_b32<0>(at, zbase);
        t.s = ring_load_b32<0>(at, sbase);
        const int64_t bsrow = (int64_t)((min(tile, ntiles - 1) * 16) >> 7) * sfull + sk0;
        const int kb = min(ks0 + (lane & 3), steps - 1);
        if constexpr (SDT == LLMK_F32) t.bs = ring_load_b32<0>((uint32_t)(bsrow + kb) * 4u, bsbase);
        else t.bs = ring_load_u16<0>((uint32_t)(bsrow + kb) * 2u, bsbase);
    };
    // how far the dword of zero points / scales of a tile was pulled back (bits): the same for every tile of a lane
    // except the last columns of the matrix
    auto pulled = [&](int tile) {
        const int n = tile < ntiles ? min(tile * 16 + r, N - 1) : 0;
        const int64_t want = (int64_t)n * sfull + sk0 + ks0, last = (int64_t)N * sfull - 4;
        return (int)(want - min(want, last)) * 8;
    };
    auto tile_wait = [&](auto nc, TileRegs& t) __attribute__((always_inline)) {
        constexpr int NY = decltype(nc)::value;
        if constexpr (ROUNDS == 1) ring_wait<NY>(t.w[0], t.w[1]);
        else ring_wait<NY>(t.w[0], t.w[1], t.w[2], t.w[3]);
        ring_wait<NY>(t.z, t.s, t.bs);
    };
    auto stage_tile = [&](const TileRegs& t, int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int hh = 0; hh < 2; ++hh)
#pragma unroll
            for (int rd = 0; rd < ROUNDS; ++rd)
                *(v4i*)(tbuf + buf * TB + hh * ROWSTRIDE + rd * 8192 + wave * 1024 + lane * 16) = t.w[hh * ROUNDS + rd];
    };

    // resident activation fragments (chunks g and g + 4 of every 128-byte step) and their scales are requested
    // first, hand-issued like the weights (an ordinary load in front of hand-issued ones would make the compiler
    // wait for all of them): the per-step sums below are computed while the first weight tiles are on their way
    v4i alo[U][MT], ahi[U][MT];
    int araw[U][MT];
    {
        typedef typename ScaleIO<SDT>::Raw SRaw;
        const RingBase abase = ring_base((const uint8_t*)p.a + k0), asbase = ring_base(p.a_s);
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int ks = min(ks0 + u, steps - 1);
                const int arow = min(m0 + 16 * mt + r, M - 1);
                const uint32_t off = (uint32_t)arow * (uint32_t)Kfull + (uint32_t)(16 * g + ks * 128);
                alo[u][mt] = ring_load_b128<0>(off, abase);
                ahi[u][mt] = ring_load_b128<64>(off, abase);
                const uint32_t soff = (uint32_t)(arow * sfull + sk0 + ks) * (uint32_t)sizeof(SRaw);
                if constexpr (sizeof(SRaw) == 4) araw[u][mt] = ring_load_b32<0>(soff, asbase);
                else araw[u][mt] = ring_load_u16<0>(soff, asbase);
            }
    }

    int tile = blockIdx.x;
    const int stride = gridDim.x;
    if (tile >= ntiles) return;
    TileRegs tr[D];
#pragma unroll
    for (int j = 0; j < D - 1; ++j) issue_tile(tr[j], tile + j * stride);

    // the activations have landed when only the loads of the two tiles just requested are in flight
    v8i afrag[U][MT];
    float ascale[U][MT];
    {
        constexpr int NY = (D - 1) * LPT;
        static_assert(U == 4 && (MT == 1 || MT == 2), "the waits below are spelled out for these sizes");
        if constexpr (MT == 1) {
            ring_wait<NY>(alo[0][0], alo[1][0], alo[2][0], alo[3][0], ahi[0][0], ahi[1][0], ahi[2][0], ahi[3][0]);
            ring_wait<NY>(araw[0][0], araw[1][0], araw[2][0], araw[3][0]);
        } else {
            ring_wait<NY>(alo[0][0], alo[1][0], alo[2][0], alo[3][0], ahi[0][0], ahi[1][0], ahi[2][0], ahi[3][0]);
            ring_wait<NY>(alo[0][MT - 1], alo[1][MT - 1], alo[2][MT - 1], alo[3][MT - 1], ahi[0][MT - 1], ahi[1][MT - 1], ahi[2][MT - 1], ahi[3][MT - 1]);
            ring_wait<NY>(araw[0][0], araw[1][0], araw[2][0], araw[3][0]);
            ring_wait<NY>(araw[0][MT - 1], araw[1][MT - 1], araw[2][MT - 1], araw[3][MT - 1]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const v4i x = alo[u][mt], y = ahi[u][mt];
                afrag[u][mt] = (v8i){x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]};
                typedef typename ScaleIO<SDT>::Raw SRaw;
                if constexpr (sizeof(SRaw) == 4) ascale[u][mt] = __int_as_float(araw[u][mt]);
                else ascale[u][mt] = ScaleIO<SDT>::cvt((SRaw)(araw[u][mt] & 0xffff));
            }
    }

#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            int sum = 0;
#pragma unroll
            for (int w = 0; w < 8; ++w) {
                const int x = afrag[u][mt][w];
                sum += (x << 24 >> 24) + (x << 16 >> 24) + (x << 8 >> 24) + (x >> 24);
            }
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            if (g == 0 && step_ok(u)) tab[(mt * 16 + r) * steps + ks0 + u] = make_float2(ascale[u][mt], (float)sum);
        }
    tile_wait(std::integral_constant<int, LPT>{}, tr[0]);          // the first tile; the second may still be on its way
    stage_tile(tr[0], 0);
    __syncthreads();
    float2 rtab[TAB_REGS ? U : 1][4];
    if constexpr (TAB_REGS) {
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) rtab[u][i] = tab[(4 * g + i) * steps + min(ks0 + u, steps - 1)];
    }

    const unsigned byte_sel = (unsigned)(col8 >> 1);
    const unsigned sel = byte_sel | ((4u + byte_sel) << 8) | 0x0c0c0000u;     // byte of this column from two words
    const int nsh = 4 * (col8 & 1);
    auto nib4 = [&](const v4i& w) {                        // this column's nibble of four consecutive words -> 4 bytes
        const unsigned t01 = __builtin_amdgcn_perm((unsigned)w[1], (unsigned)w[0], sel);
        const unsigned t23 = __builtin_amdgcn_perm((unsigned)w[3], (unsigned)w[2], sel);
        return (int)((__builtin_amdgcn_perm(t23, t01, 0x05040100u) >> nsh) & 0x0f0f0f0fu);
    };

    v4f acc[MT];
    auto clear_acc = [&]() {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[mt] = (v4f){0.f, 0.f, 0.f, 0.f};
    };
    clear_acc();
    int parity = 0;

    auto load_q = [&](const uint8_t* row, int ksc, v4i& ql, v4i& qh) __attribute__((always_inline)) {
        const v4i* wl = (const v4i*)(row + (ksc * 128 + 16 * g) * 4);
        const v4i* wh = (const v4i*)(row + (ksc * 128 + 64 + 16 * g) * 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) { ql[i] = nib4(wl[i]); qh[i] = nib4(wh[i]); }
    };
    auto row_entry = [&](int u, int mt, int i, int ksc) __attribute__((always_inline)) {
        if constexpr (TAB_REGS) return rtab[u][i];
        else return tab[(mt * 16 + 4 * g + i) * steps + ksc];
    };
    // raw nibbles through the MFMA, zero point and scale applied to the 128-K partial sums: every partial
    // is an integer below 2^24, so the fp32 arithmetic up to the scale product is exact
    auto step_fast = [&](int u, int ksc, const v4i& ql, const v4i& qh, int z, int sc4, float bs) __attribute__((always_inline)) {
        const float zf = (float)z, c1 = bs * (float)sc4;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const v8i a = afrag[u][mt];
            v4i pr = {0, 0, 0, 0};
            pr = mfma_i8_16x16x64((v4i){a[0], a[1], a[2], a[3]}, ql, pr);
            pr = mfma_i8_16x16x64((v4i){a[4], a[5], a[6], a[7]}, qh, pr);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float2 e = row_entry(u, mt, i, ksc);
                const float part = fmaf(-zf, e.y, (float)pr[i]);
                acc[mt][i] = fmaf(part, c1 * e.x, acc[mt][i]);
            }
        }
    };
    // exact int8 wrap of (q - z) and of the product, nibble by nibble
    auto step_wrap = [&](int u, int ksc, const v4i& ql, const v4i& qh, int z, int sc4, float bs) __attribute__((always_inline)) {
        auto deq4 = [&](int q4) {
            unsigned o = 0;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int q = (q4 >> (8 * b)) & 0xf;
                const int d = (int)(int8_t)(q - z);
                o |= ((unsigned)((d * sc4) & 0xff)) << (8 * b);
            }
            return (int)o;
        };
        v4i bl, bh;
#pragma unroll
        for (int i = 0; i < 4; ++i) { bl[i] = deq4(ql[i]); bh[i] = deq4(qh[i]); }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const v8i a = afrag[u][mt];
            v4i pr = {0, 0, 0, 0};
            pr = mfma_i8_16x16x64((v4i){a[0], a[1], a[2], a[3]}, bl, pr);
            pr = mfma_i8_16x16x64((v4i){a[4], a[5], a[6], a[7]}, bh, pr);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float2 e = row_entry(u, mt, i, ksc);
                acc[mt][i] = fmaf((float)pr[i], bs * e.x, acc[mt][i]);
            }
        }
    };
    auto mul_tile = [&](const TileRegs& t, int buf) __attribute__((always_inline)) {
        const uint8_t* row = tbuf + buf * TB + half * ROWSTRIDE;
        bool ok[U], all_ok = true;
        float bs[U];
        int ksc[U], zu[U], su[U];
        const int sh = pulled(tile);
        const unsigned tz = sh < 32 ? (unsigned)t.z >> sh : 0u, ts = sh < 32 ? (unsigned)t.s >> sh : 0u;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            ksc[u] = min(ks0 + u, steps - 1);
            const int z = (int)(tz << (24 - 8 * u)) >> 24, sc4 = (int)(ts << (24 - 8 * u)) >> 24;
            zu[u] = z;
            su[u] = sc4;
            // (q - z) * s for q = 0 and q = 15 bound every product of the group (24-bit multiplies are exact here)
            const int p0 = -__mul24(z, sc4), p15 = p0 + 15 * sc4;
            ok[u] = z >= -112 && min(p0, p15) >= -128 && max(p0, p15) <= 127;
            all_ok = all_ok && ok[u];
            const unsigned raw = (unsigned)__builtin_amdgcn_readlane((int)t.bs, u);
            if constexpr (SDT == LLMK_F32) bs[u] = __uint_as_float(raw);
            else bs[u] = ScaleIO<SDT>::cvt((unsigned short)raw);
            if (!step_ok(u)) bs[u] = 0.f;
        }
        if (__builtin_amdgcn_ballot_w64(!all_ok) == 0) {
            // one straight-line block for the whole tile: the LDS reads of a step overlap the arithmetic of the one before
            v4i ql[2], qh[2];
            load_q(row, ksc[0], ql[0], qh[0]);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (u + 1 < U) load_q(row, ksc[u + 1], ql[(u + 1) & 1], qh[(u + 1) & 1]);
                step_fast(u, ksc[u], ql[u & 1], qh[u & 1], zu[u], su[u], bs[u]);
            }
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                v4i ql, qh;
                load_q(row, ksc[u], ql, qh);
                if (__builtin_amdgcn_ballot_w64(!ok[u]) == 0) step_fast(u, ksc[u], ql, qh, zu[u], su[u], bs[u]);
                else step_wrap(u, ksc[u], ql, qh, zu[u], su[u], bs[u]);
            }
        }
    };
    // cross-wave reduction and store of the finished tile; the same barrier publishes the next tile's bytes
    auto finish = [&](auto stage_c, int tl, const TileRegs& next, int next_buf) __attribute__((always_inline)) {
        float* rbuf = red + parity * NW * MT * 256;
        parity ^= 1;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) *(v4f*)(rbuf + ((wave * MT + mt) * 64 + lane) * 4) = acc[mt];
        if constexpr (decltype(stage_c)::value) stage_tile(next, next_buf);
        __syncthreads();
        const int n0 = tl * 16;
        for (int o = tid; o < MT * 256; o += NW * 64) {
            const int mt = o >> 8, row16 = (o & 255) >> 4, col = o & 15;
            const int src = (mt * 64 + (row16 >> 2) * 16 + col) * 4 + (row16 & 3);
            const int m = m0 + 16 * mt + row16, n = n0 + col;
            if (m >= M || n >= N) continue;
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) sum += rbuf[w * MT * 256 + src];
            if (p.partial) p.partial[((int64_t)blockIdx.z * M + m) * N + n] = sum;
            else st_out(p.c, (int64_t)m * N + n, sum, p.c_dtype);
        }
        clear_acc();
    };
    // Slot d of the ring: request tile i + 2 into the set that tile i - 1 has left, multiply tile i (its words are in
    // LDS, staged by the slot before), wait for tile i + 1 (only the LPT loads just requested are younger), and
    // finish: reduce and store tile i while the same barrier publishes the staged words of tile i + 1.  Whole rounds
    // of the three slots run in a loop without a branch (requests past the last tile are clamped).  Behind the loop
    // everything requested is waited for, consumed or not, and the remaining one or two tiles request nothing: a
    // register whose load nobody consumes would be reused by the compiler while the load is still in flight.
    int lbuf = 0;
    const std::true_type yes;
    const std::false_type no;
    auto slot = [&](auto dc) __attribute__((always_inline)) {
        constexpr int d = decltype(dc)::value;
        issue_tile(tr[(d + 2) % D], tile + (D - 1) * stride);
        mul_tile(tr[d], lbuf);
        tile_wait(std::integral_constant<int, LPT>{}, tr[(d + 1) % D]);
        finish(yes, tile, tr[(d + 1) % D], lbuf ^ 1);
        lbuf ^= 1;
        tile += stride;
    };
    static_assert(D == 3, "ring slots are spelled out below");
    const int my_tiles = (ntiles - tile + stride - 1) / stride;
    for (int rd = my_tiles / D; rd > 0; --rd) {
        slot(std::integral_constant<int, 0>{});
        slot(std::integral_constant<int, 1>{});
        slot(std::integral_constant<int, 2>{});
    }
    tile_wait(std::integral_constant<int, 0>{}, tr[1]);
    const int rem = my_tiles % D;
    if (rem > 0) {
        mul_tile(tr[0], lbuf);
        if (rem > 1) {
            finish(yes, tile, tr[1], lbuf ^ 1);
            lbuf ^= 1;
            tile += stride;
            mul_tile(tr[1], lbuf);
        }
        finish(no, tile, tr[1], lbuf);
    }
}

template <int MT, int SDT>
int launch_w4a8_stream(W4A8Args p, void* workspace, int64_t workspace_bytes, hipStream_t st) {
    // K ranges of at most 4096 elements, equally long up to one step
    const int steps_all = p.K >> 7, nz = (steps_all + 31) / 32;
    p.Kc = ((steps_all + nz - 1) / nz) * 128;
    p.partial = nullptr;
    if (nz > 1) {
        if (!workspace || workspace_bytes < (int64_t)nz * p.M * p.N * 4 || (((uintptr_t)workspace) & 15))
            LLMK_FAIL(LLMK_ERR_ARG, "gemm_w4a8: K > 4096 needs %lld bytes of 16-byte aligned workspace", (long long)nz * p.M * p.N * 4);
        p.partial = (float*)workspace;
    }
    const int steps = p.Kc >> 7, rounds = p.Kc * 4 > 8192 ? 2 : 1;
    const int ntiles = (p.N + 15) >> 4, mtiles = (p.M + 16 * MT - 1) / (16 * MT);
    const size_t smem = (size_t)2 * 8 * MT * 256 * 4 + (size_t)MT * 16 * steps * 8 + (size_t)2 * 2 * (rounds * 8192 + 64);
    auto k1 = w4a8_stream_kernel<MT, SDT, 1>;
    auto k2 = w4a8_stream_kernel<MT, SDT, 2>;
    static std::atomic<uint64_t> cfg1{0}, cfg2{0};
    if (int rc = llmk_reserve_lds((const void*)k1, 160 * 1024, cfg1, "gemm_w4a8")) return rc;
    if (int rc = llmk_reserve_lds((const void*)k2, 160 * 1024, cfg2, "gemm_w4a8")) return rc;
    const int cus = llmk_device_cus();
    if (cus <= 0) LLMK_FAIL(LLMK_ERR_LAUNCH, "gemm_w4a8: cannot query the device");
    const int rows = mtiles * nz;                                      // workgroup rows that share the column tiles
    int gx = min(ntiles, max(1, cus / min(rows, cus)));                // one workgroup per CU (LDS bound)
    { const int per_wg = (ntiles + gx - 1) / gx; gx = (ntiles + per_wg - 1) / per_wg; }   // equal tile counts
    dim3 grid((unsigned)gx, (unsigned)mtiles, (unsigned)nz);
    if (rounds == 1) k1<<<grid, 512, smem, st>>>(p);
    else k2<<<grid, 512, smem, st>>>(p);
    LLMK_CHECK_LAUNCH("gemm_w4a8(stream)");
    if (nz > 1) {
        const int64_t mn = (int64_t)p.M * p.N;
        const unsigned blocks = (unsigned)cdiv64(cdiv64(mn, 4), 256);
        if (p.c_dtype == LLMK_BF16) splitk_sum_kernel<LLMK_BF16><<<blocks, 256, 0, st>>>(p.partial, p.c, mn, nz);
        else if (p.c_dtype == LLMK_F16) splitk_sum_kernel<LLMK_F16><<<blocks, 256, 0, st>>>(p.partial, p.c, mn, nz);
        else splitk_sum_kernel<LLMK_F32><<<blocks, 256, 0, st>>>(p.partial, p.c, mn, nz);
        LLMK_CHECK_LAUNCH("gemm_w4a8(sum)");
    }
    return LLMK_OK;
}

}  // namespace

// Which path a shape takes (pointer alignment aside) and the scratch that path uses.
namespace {
struct W4A8Plan {
    bool stream;          // fused decode kernel
    bool tiles;           // 128-column tile kernels that expand the packed words themselves
    int64_t nz;           // K ranges of the decode kernel
    int64_t bytes;        // scratch the chosen path uses
};
// scratch layout of the two-pass path: int8 copy of W | fp32 activation scales | fp32 weight scales | the int8 GEMM's own
inline int64_t w4a8_two_pass_scales_off(int64_t N, int64_t K) { return (N * K + 255) & ~(int64_t)255; }
inline int64_t w4a8_a_s32_bytes(int64_t M, int64_t K) { return (M * (K / 128) * 4 + 255) & ~(int64_t)255; }
inline int64_t w4a8_widened_bytes(int64_t M, int64_t N, int64_t K) {
    return w4a8_a_s32_bytes(M, K) + ((((N + 127) / 128) * (K / 128) * 4 + 255) & ~(int64_t)255);
}

W4A8Plan w4a8_plan(int64_t M, int64_t N, int64_t K, int group_int4) {
    W4A8Plan pl{false, false, 1, 0};
    if (M <= 0 || N <= 0 || K <= 0) return pl;
    // Measured on MI355X with x = N * K / 4096^2: the fused kernel takes about 5 + 3.4 x microseconds per 32 rows
    // of M; expanding to int8 and running the int8 GEMM about 26 + 3.6 x for x <= 4 and more beyond.
    const double x = (double)N * (double)K / (4096.0 * 4096.0);
    const int64_t row_blocks = (M + 31) / 32;
    const bool fused_wins = row_blocks <= 2 || (row_blocks == 3 && x <= 3.0) || (row_blocks == 4 && x <= 2.0);
    // K > 4096 runs as ranges of at most 4096 with fp32 partial sums in the workspace (up to 64 rows)
    pl.nz = (K / 128 + 31) / 32;
    const bool long_k_ok = pl.nz == 1 || row_blocks <= 2;
    // (the hand-issued loads of the fused kernel take 32-bit lane offsets into the activations and the tables)
    const bool small_offsets = M * K < (1ll << 32) && N * (K / 128) < (1ll << 32);
    // 65 to 256 rows on at most one 64-column workgroup per CU: the tile kernel with 512-byte K steps
    const bool mid = M > 64 && M <= 256 && mid_plan(M, N, K).tiles <= LLMK_CUS && K <= 16384;
    pl.stream = fused_wins && long_k_ok && small_offsets && group_int4 == 128 && !mid;
    // Mid-size M: the tile kernels unpack and dequantise inside their K loop (one pass over the packed words; the
    // separate expansion writes and re-reads N * K bytes).  Measured (us per launch, fused | expansion + int8 GEMM):
    // the 64-column kernel with 512-byte K steps on at most one workgroup per CU: 256 x 4096 x 4096 19.4 | 29.8,
    // 256 x 4096 x 14336 54.2 | 60.6; the 128-column kernel up to 128 rows: 128 x 14336 x 4096 40.5 | 44.6,
    // 128 x 4096 x 14336 41.2 | 46.5; from there on the two passes win (512 x 4096 x 4096 34 | 30, 512 x 14336 x 4096 80 | 60).
    DirectArgs q{};
    q.M = (int)M; q.N = (int)N; q.K = (int)K;
    pl.tiles = !pl.stream && M > 64 && (mid || M <= 128) && group_int4 == 128 && N <= 0x7fffffff &&
               K <= 0x7fffffff && dma_eligible(q);
    if (pl.stream) pl.bytes = pl.nz > 1 ? pl.nz * M * N * 4 : 0;
    else if (pl.tiles) pl.bytes = llmk_gemm_workspace_bytes(M, N, K);      // fp32 activation scales + split-K partial sums
    else pl.bytes = w4a8_two_pass_scales_off(N, K) + w4a8_widened_bytes(M, N, K) + llmk_gemm_workspace_bytes(M, N, K);
    return pl;
}

// The tile path: 16-bit activation scales are widened into the workspace first (the pipeline streams 4-byte
// scale elements), few tiles split K over workgroups with fp32 partial sums behind them.
int launch_w4a8_tiles(DirectArgs p, void* workspace, int64_t workspace_bytes, hipStream_t stream) {
    const char* name = "gemm_w4a8(fused tiles)";
    // the 64-column kernel takes 16-bit activation scales as they are
    if (p.M <= 256 && mid_plan(p.M, p.N, p.K).tiles <= LLMK_CUS && p.K <= 16384) {
        MidPlan pl = mid_plan(p.M, p.N, p.K);
        if (pl.z > 1 && workspace_bytes < (int64_t)pl.z * p.M * p.N * 4) pl.z = 1;
        if (mid_eligible<K_W4A8>(p, pl.mt, pl.z)) {
            if (pl.z > 1) { p.partial = (float*)workspace; p.ksplit = pl.z; }
            if (p.s_dtype != LLMK_F32)
                return pl.mt == 4 ? launch_mid<K_W4A8, 4, true>(p, stream, name) : launch_mid<K_W4A8, 2, true>(p, stream, name);
            return pl.mt == 4 ? launch_mid<K_W4A8, 4>(p, stream, name) : launch_mid<K_W4A8, 2>(p, stream, name);
        }
    }
    // the 128-column kernels stage 16-bit scales as they are, too
    const int64_t used = 0;
    const int z = splitk_factor(p.M, p.N, p.K);
    if (z > 1 && workspace_bytes - used >= (int64_t)z * p.M * p.N * 4) {
        p.partial = (float*)((uint8_t*)workspace + used);
        p.ksplit = z;
    }
    if (p.s_dtype != LLMK_F32) return launch_dma<K_W4A8, false, true>(p, stream, name);
    return launch_dma<K_W4A8, false>(p, stream, name);
}
}  // namespace

extern "C" int64_t llmk_gemm_w4a8_workspace_bytes(int64_t M, int64_t N, int64_t K, int group_int4) {
    return w4a8_plan(M, N, K, group_int4).bytes;
}

extern "C" int llmk_gemm_w4a8(const int8_t* a, const void* a_s, const int32_t* b_packed, const void* b_s, int s_dtype,
                              const int8_t* b_s4, const int8_t* b_z4, void* c, int c_dtype, int64_t M, int64_t N,
                              int64_t K, int group_int4, void* workspace, int64_t workspace_bytes, void* stream) {
    if (M < 0 || N < 0 || K < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a8: negative dimension");
    if (K % 128 || N % 8) LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a8: need K %% 128 == 0 and N %% 8 == 0 (K=%lld N=%lld)", (long long)K, (long long)N);
    if (group_int4 < 4 || group_int4 % 4 || K % group_int4) LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a8: group_int4=%d must divide K and be a multiple of 4", group_int4);
    if (M == 0 || N == 0) return LLMK_OK;
    if (!a || !a_s || !b_packed || !b_s || !b_s4 || !b_z4 || !c) LLMK_FAIL(LLMK_ERR_ARG, "gemm_w4a8: null pointer");
    const W4A8Plan pl = w4a8_plan(M, N, K, group_int4);
    const bool ranges_ok = pl.nz == 1 || (workspace && workspace_bytes >= pl.nz * M * N * 4 && !(((uintptr_t)workspace) & 15));
    if (pl.stream && ranges_ok && !(((uintptr_t)a | (uintptr_t)b_packed) & 15)) {
        W4A8Args p{a, a_s, b_packed, b_s, b_s4, b_z4, c, c_dtype, (int)M, (int)N, (int)K, 0, nullptr};
        if (c_dtype != LLMK_F32 && c_dtype != LLMK_F16 && c_dtype != LLMK_BF16) LLMK_FAIL(LLMK_ERR_DTYPE, "gemm_w4a8: c_dtype %d", c_dtype);
        hipStream_t st = (hipStream_t)stream;
#define LLMK_W4A8_MT(SDT)                                                    \
        do {                                                                 \
            /* 16-row workgroups side by side win while the weights are small, 32-row ones beyond */ \
            if (M <= 16 || N * K <= ((int64_t)20 << 20)) return launch_w4a8_stream<1, SDT>(p, workspace, workspace_bytes, st); \
            return launch_w4a8_stream<2, SDT>(p, workspace, workspace_bytes, st); \
        } while (0)
        if (s_dtype == LLMK_F16) LLMK_W4A8_MT(LLMK_F16);
        if (s_dtype == LLMK_BF16) LLMK_W4A8_MT(LLMK_BF16);
        if (s_dtype == LLMK_F32) LLMK_W4A8_MT(LLMK_F32);
#undef LLMK_W4A8_MT
        LLMK_FAIL(LLMK_ERR_DTYPE, "gemm_w4a8: s_dtype %d", s_dtype);
    }
    if (pl.tiles && !(((uintptr_t)a | (uintptr_t)b_packed | (uintptr_t)workspace) & 15)) {
        if (!workspace) workspace_bytes = 0;                // no scratch: no K split, everything else as with it
        if (s_dtype != LLMK_F32 && s_dtype != LLMK_F16 && s_dtype != LLMK_BF16) LLMK_FAIL(LLMK_ERR_DTYPE, "gemm_w4a8: s_dtype %d", s_dtype);
        if (c_dtype != LLMK_F32 && c_dtype != LLMK_F16 && c_dtype != LLMK_BF16) LLMK_FAIL(LLMK_ERR_DTYPE, "gemm_w4a8: c_dtype %d", c_dtype);
        DirectArgs p{};
        p.a = (const uint8_t*)a; p.b = (const uint8_t*)b_packed; p.c = c; p.a_s = a_s; p.b_s = b_s;
        p.w4_s4 = b_s4; p.w4_z4 = b_z4;
        p.c_dtype = c_dtype; p.s_dtype = s_dtype; p.M = (int)M; p.N = (int)N; p.K = (int)K; p.E = 1; p.group = 128;
        return launch_w4a8_tiles(p, workspace, workspace_bytes, (hipStream_t)stream);
    }
    if (!workspace || workspace_bytes < N * K) LLMK_FAIL(LLMK_ERR_ARG, "gemm_w4a8: workspace of N*K=%lld bytes required", (long long)(N * K));
    // 16-bit block scales are widened by spare blocks of the expansion launch when the scratch has room for them
    W4A8Widen wd{};
    int64_t used = (N * K + 15) & ~(int64_t)15;
    const int64_t soff = w4a8_two_pass_scales_off(N, K);
    if ((s_dtype == LLMK_F16 || s_dtype == LLMK_BF16) && K > 0 && !((uintptr_t)workspace & 255) &&
        workspace_bytes >= soff + w4a8_widened_bytes(M, N, K)) {
        wd.a_s = a_s; wd.b_s = b_s; wd.s_dtype = s_dtype;
        wd.n_a = M * (K / 128); wd.n_b = ((N + 127) / 128) * (K / 128);
        wd.a_s32 = (float*)((uint8_t*)workspace + soff);
        wd.b_s32 = (float*)((uint8_t*)workspace + soff + w4a8_a_s32_bytes(M, K));
        used = soff + w4a8_widened_bytes(M, N, K);
    }
    if (K > 0) {
        const unsigned expand_blocks = (unsigned)cdiv64((N / 8) * (K / 4), 256);
        unsigned blocks = expand_blocks;
        if (wd.a_s32) {
            wd.first_block = expand_blocks;
            blocks += (unsigned)cdiv64(wd.n_a + wd.n_b, 256);
        }
        w4a8_expand_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>(b_packed, b_s4, b_z4, (int8_t*)workspace, N, K, group_int4, wd);
        LLMK_CHECK_LAUNCH("gemm_w4a8(expand)");
    }
    // what is left of the workspace behind the expanded weights (16-byte aligned) serves the int8 GEMM
    void* rest = workspace_bytes > used ? (void*)((uint8_t*)workspace + used) : nullptr;
    const int64_t rest_bytes = rest ? workspace_bytes - used : 0;
    if (wd.a_s32)
        return llmk_gemm_i8_block(a, wd.a_s32, (const int8_t*)workspace, wd.b_s32, LLMK_F32, c, c_dtype, M, N, K, rest, rest_bytes, stream);
    return llmk_gemm_i8_block(a, a_s, (const int8_t*)workspace, b_s, s_dtype, c, c_dtype, M, N, K, rest, rest_bytes, stream);
}
