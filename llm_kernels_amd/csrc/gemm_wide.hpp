// 256 x 256 output tile variant of the direct-to-LDS pipeline, for problems large enough to fill the
// chip with such tiles.  Per K step a workgroup moves (256 + 256) x 128 bytes from L2 to LDS for
// 256 x 256 x 128 multiply-adds: a third less L2 and a quarter less LDS traffic per flop than the
// 256 x 128 tile, which is what bounds that kernel.
//
// Workgroup: 512 threads = 8 waves, 2 along M x 4 along N; wave tile 128 rows x 64 columns =
// 8 x 4 MFMA tiles (128 accumulator registers per lane).  Two LDS stages of 66560 bytes
// (A 32 KB, B 32 KB, activation-scale column 1 KB).  A step has two barriers: one in the middle, behind
// which the weight rows of K step kt+2 are requested (every wave holds the weight fragments of step kt in
// registers by then), and one before its last tile row, behind which the activation rows of step kt+2 are
// requested and the fragments of step kt+1 fetched; the loads fly while step kt+1 is multiplied.
//
// Inside a step a wave keeps its four weight fragments in registers for the whole step and streams
// the eight activation fragments through a two-deep register buffer.  The product of tile n is
// scaled and accumulated (VALU) while the MFMAs of the next tile row run, through two register sets
// of partial products that carry over from one K step to the next.
#pragma once
#include <type_traits>
#include "gemm_mid.hpp"
#include "quant_util.hpp"

namespace llmk {

// R = tile rows (of 16) per wave: 8 gives the 256 x 256 tile described above, 4 a 128 x 256 tile (wave tile
// 64 x 64) with the same loop for problems with too few rows for a round of the large tile.
constexpr int W_BN = 256, W_THREADS = 512;
constexpr int W_B = W_BN * 128, W_S = 256 * 4;
constexpr int w_bm(int r) { return 32 * r; }
constexpr int w_stage(int r) { return w_bm(r) * 128 + W_B + W_S; }        // 66560 / 50176
constexpr int w_lds(int r) { return 2 * w_stage(r) + 2 * D_MAX_KT * 4; }  // 135168 / 102400 bytes

// ---- which tile a workgroup works on.  `lin` = linear workgroup id (blockIdx.y * gridDim.x + blockIdx.x), gx = column
// tiles.  Workgroups go to the eight XCDs round robin by linear id, each XCD with its own L2, and 256 of them (one
// per CU) run at a time.
struct WideTile {
    int bx, m_start, m_end, e;
    bool found;
};

template <bool GROUPED, int R>
__device__ __forceinline__ WideTile wide_tile_of(const DirectArgs& p, int lin, int gx) {
    constexpr int W_BM = w_bm(R);
    WideTile t;
    t.e = 0;
    t.found = false;
    if constexpr (!GROUPED) {
        // Within every round of 256 workgroups give each XCD a compact block of 8 x 4 tiles of one strip of four
        // tile rows instead of every eighth tile of the grid, so that its L2 holds few operand rows and all XCDs of
        // a round share the four activation row tiles.
        const int gy = (p.M + W_BM - 1) / W_BM, total = gx * gy;
        if (lin >= total) return t;
        int bx = lin % gx, by = lin / gx;
        constexpr int H = 4;      // strips of 8 or 16 tile rows measured 1-13 % slower
        if (gy % H == 0) {
            int lp = lin;
            if (lin < (total & ~(LLMK_CUS - 1))) {
                const int w = lin & (LLMK_CUS - 1);
                lp = (lin & ~(LLMK_CUS - 1)) + (w & 7) * (LLMK_CUS / 8) + (w >> 3);
            }
            const int strip = lp / (H * gx), rr = lp % (H * gx);
            bx = rr / H;
            by = strip * H + rr % H;
        }
        t.bx = bx;
        t.m_start = by * W_BM;
        t.m_end = min(p.M, t.m_start + W_BM);
        t.found = true;
    } else {
        int e = 0;
        int64_t s0 = p.seg_indptr[0];
        if (gx % 8 == 0) {
            // XCD x (workgroup id mod 8) owns the column tiles x, x + 8, ...; it walks them segment by
            // segment, and for every column tile the row tiles of the segment back to back, so the workgroups
            // that share a weight tile run at the same time on the L2 that holds it.  Long segments go in strips of
            // four row tiles (the last strip takes what is left, one to five), each strip across all column tiles
            // of the XCD: its 32 concurrent workgroups then share 8 weight tiles and 4 activation tiles, where one
            // column tile x 32 row tiles would pull 33 operand tiles per K step through the L2 instead of 12.
            const int x = lin & 7, cx = gx >> 3;
            int s = lin >> 3;
            for (; e < p.E; ++e) {
                const int64_t s1 = p.seg_indptr[e + 1];
                const int tl = (int)((s1 - s0 + W_BM - 1) / W_BM);
                if (s < tl * cx) {
                    const int full = max(1, (tl + 2) >> 2) - 1;          // strips of four in front of the last one
                    int bl, rt;
                    if (s < 4 * cx * full) {
                        const int st = s / (4 * cx), r4 = s - st * 4 * cx;
                        bl = r4 >> 2;
                        rt = 4 * st + (r4 & 3);
                    } else {
                        const int r4 = s - 4 * cx * full, h = tl - 4 * full;
                        bl = r4 / h;
                        rt = 4 * full + (r4 - bl * h);
                    }
                    t.found = true;
                    t.bx = bl * 8 + x;
                    t.m_start = (int)s0 + rt * W_BM;
                    t.m_end = min((int)s1, t.m_start + W_BM);
                    break;
                }
                s -= tl * cx;
                s0 = s1;
            }
        } else {
            int tile = lin / gx, cum = 0;
            t.bx = lin % gx;
            for (; e < p.E; ++e) {
                const int64_t s1 = p.seg_indptr[e + 1];
                const int tl = (int)((s1 - s0 + W_BM - 1) / W_BM);
                if (tile < cum + tl) { t.found = true; t.m_start = (int)s0 + (tile - cum) * W_BM; t.m_end = min((int)s1, t.m_start + W_BM); break; }
                cum += tl;
                s0 = s1;
            }
        }
        t.e = e;
    }
    return t;
}

// number of tiles of the launch (the valid linear ids are 0 .. total - 1 under both orders above)
template <bool GROUPED, int R>
__device__ __forceinline__ int wide_total_tiles(const DirectArgs& p, int gx) {
    constexpr int W_BM = w_bm(R);
    if constexpr (!GROUPED) return gx * ((p.M + W_BM - 1) / W_BM);
    int rows = 0;
    int64_t s0 = p.seg_indptr[0];
    for (int e = 0; e < p.E; ++e) {
        const int64_t s1 = p.seg_indptr[e + 1];
        rows += (int)((s1 - s0 + W_BM - 1) / W_BM);
        s0 = s1;
    }
    return rows * gx;
}

// A launch of `total` tiles runs in rounds of 256 (one workgroup per CU).  When the last round holds at most 128
// tiles, each of them is split along K into z = 256 / ntail (at most 8) work items of ktz K steps (even, at least
// eight), which write fp32 partial sums that wide_tail_sum_kernel adds: the round then takes 1 / z of a tile's
// time instead of all of it with most of the chip idle.  The split is taken when the time it saves (a K step
// costs about 1.6 us) is at least 1.5 times what the partial sums cost (0.5 MB written and read per work item at
// 5 TB/s, plus 6 us for the second kernel) and K has at least 64 steps (8192 bytes; with fewer steps a tile is too
// short for the split to pay: measured on the Mixtral gate/up projection, 955 -> 985 us).  z == 1: no split.
struct WideTail {
    int full, ntail, z, ktz;
};
constexpr int W_TAIL_MIN_KT = 64;
__host__ __device__ inline WideTail wide_tail_plan(int total, int KT) {
    WideTail w;
    w.full = total & ~(LLMK_CUS - 1);
    w.ntail = total - w.full;
    w.z = 1;
    w.ktz = KT;
    if (w.ntail > 0 && w.ntail <= LLMK_CUS / 2 && KT >= W_TAIL_MIN_KT) {
        int z = LLMK_CUS / w.ntail;
        if (z > 8) z = 8;
        int ktz = ((KT + z - 1) / z + 1) & ~1;
        if (ktz < 8) ktz = 8;
        z = (KT + ktz - 1) / ktz;
        const int saved_x10 = KT * 16 * (z - 1) / z, cost_x10 = w.ntail * z + 60;      // tenths of a microsecond
        if (z > 1 && 2 * saved_x10 >= 3 * cost_x10) {
            w.ktz = ktz;
            w.z = z;
        }
    }
    return w;
}
constexpr int W_TAIL_ITEMS = LLMK_CUS;          // upper bound of ntail * z

// SWIGLU (grouped gate / up projection of a gated MLP, weights [E, 2 I, K] with the I gate rows first): the tile's 256
// columns are gate columns n0 .. n0 + 127 and up columns I + n0 .. I + n0 + 127 (n0 = 128 blockIdx.x), and instead of
// storing them the workgroup applies the gated activation and the 1 x 128 activation quantiser of the next projection:
// p.c receives [M, I] quantised values, p.q_scale their scales.  Every rounding point of the separate kernels is kept
// (sums rounded to the tensor dtype p.c_dtype, activation and product in that dtype, the quantiser's own arithmetic), so
// the outputs equal those of GEMM + activation + quantiser bit for bit; the [M, 2 I] tensor never exists.
template <int KIND, bool GROUPED, int R = 8, bool SWIGLU = false>
__global__ __launch_bounds__(W_THREADS) void gemm_wide_kernel(DirectArgs p) {
    constexpr bool AS16 = false;             // 16-bit activation scales are widened before this kernel, see launch_big
    static_assert(R == 8 || R == 4, "tile rows per wave");
    static_assert(!SWIGLU || (GROUPED && (KIND == K_FP8_BLOCK || KIND == K_I8_BLOCK)), "gated epilogue: grouped block-scaled kinds");
    constexpr int W_BM = w_bm(R), W_A = W_BM * 128, W_STAGE = w_stage(R);
    constexpr int AL = R / 2;                    // activation loads per thread and stage
    constexpr int W_EARLY_ROW = R == 8 ? 5 : 2;  // tile row in front of which the mid-step barrier sits
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int wm = wave >> 2, wn = wave & 3;
    constexpr bool SCALED = (KIND == K_FP8_BLOCK || KIND == K_I8_BLOCK);
    // 4-bit weights (fp16 activations): the weight rows of a stage are not loaded into LDS but expanded there by
    // the threads themselves from packed words that travel HBM -> registers, see w4_request / w4_expand
    constexpr bool W4NK = (KIND == K_W4NK), W4 = W4NK;
    static_assert(KIND != K_W4MARLIN && KIND != K_W4A8 && !(W4 && GROUPED), "4-bit weights: row-packed fp16 layout, dense launches only");
    constexpr int ESZ = (KIND == K_F16 || KIND == K_BF16 || W4) ? 2 : 1;
    const int N = p.N;
    const int K = p.K * ESZ;                 // row length in bytes
    const int KT_all = K >> 7;
    // K steps [kt0, kt0 + KT) of the tile; a work item of a split last round writes fp32 sums to `part`
    int kt0 = 0, KT = KT_all;
    float* part = nullptr;
    const int gx = gridDim.x;
    int lin = blockIdx.y * gx + blockIdx.x;
    // calibration runs only: the shader clock this workgroup saw (ticks of the core clock per tick of the 100 MHz clock)
    const bool clocked = p.clocks && lin == 0 && tid == 0;
    long long clk0 = 0, wall0 = 0;
    if (clocked) { clk0 = clock64(); wall0 = wall_clock64(); }
    WideTile wt = wide_tile_of<GROUPED, R>(p, lin, gx);
    if (p.tail_split) {
        // (the tiles of all but the last round need nothing of this: for them the plan only confirms lin < full;
        // the segment pointers it reads are the ones the lookup above has just read)
        const int total = wide_total_tiles<GROUPED, R>(p, gx);
        const WideTail tp = wide_tail_plan(total, KT_all);
        if (lin >= tp.full && tp.z > 1) {
            const int j = lin - tp.full, kpart = j / tp.ntail, idx = j - kpart * tp.ntail;
            if (kpart >= tp.z) return;
            lin = tp.full + idx;
            kt0 = kpart * tp.ktz;
            KT = min(tp.ktz, KT_all - kt0);
            part = p.partial + (int64_t)(kpart * tp.ntail + idx) * (W_BM * W_BN);
            wt = wide_tile_of<GROUPED, R>(p, lin, gx);
        }
    }
    if (!wt.found) return;
    const int bx = wt.bx, m_start = wt.m_start, m_end = wt.m_end;
    const uint8_t* bbase = p.b;
    int64_t bs_off = 0;
    if constexpr (GROUPED) {
        const int64_t widx = p.weight_indices ? p.weight_indices[wt.e] : wt.e;
        bbase += widx * (int64_t)N * K;
        bs_off = widx * (int64_t)((N + 127) / 128) * KT_all;
    }
    const int n0 = bx * (SWIGLU ? 128 : W_BN);
    const int I_half = N >> 1;               // SWIGLU: gate rows [0, I), up rows [I, 2 I) of the weight matrix

    // weight scales of the tile's two 128-column blocks, for every K step
    float* bsl = (float*)(lds + 2 * W_STAGE);
    const int nblk = (N + 127) / 128;

    // ---- source offsets of the 9 loads of a stage.  Load i of a wave fills LDS rows 8q .. 8q+7,
    // q = 4*wave + i.  A: LDS row R holds tile row R.  B: within each 64-row group, LDS row rho holds
    // tile column 32*(rho >> 5) + 8*((rho & 15) >> 2) + 4*((rho >> 4) & 1) + (rho & 3), so that MFMA j yields,
    // in lane group g, the four columns 32*(j >> 1) + 8g + 4*(j & 1) + (0..3): a lane ends up with two runs
    // of 8 consecutive columns of a row, and the four lane groups of a row write 64 contiguous bytes per
    // store instruction (1-2 % faster than 16 columns per lane, whose stores leave 16-byte gaps).
    // The 16-byte chunk index is XOR-swizzled with ((R >> 1) & 7) on the global side.
    const int row8 = lane >> 3;
    uint32_t aoff[AL], boff[4];
#pragma unroll
    for (int i = 0; i < AL; ++i) {
        const int row = 8 * (wave * AL + i) + row8;
        const uint32_t chunk = (uint32_t)((lane & 7) ^ ((row >> 1) & 7)) * 16u;
        aoff[i] = (uint32_t)min(m_start + row, m_end - 1) * (uint32_t)K + chunk;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = 8 * (wave * 4 + i) + row8;
        const uint32_t chunk = (uint32_t)((lane & 7) ^ ((row >> 1) & 7)) * 16u;
        const int rho = row & 63;
        const int col = (row & 192) + 32 * (rho >> 5) + 8 * ((rho & 15) >> 2) + 4 * ((rho >> 4) & 1) + (rho & 3);
        const int wrow = SWIGLU ? (col < 128 ? n0 + col : I_half + n0 + col - 128) : min(n0 + col, N - 1);
        boff[i] = (uint32_t)wrow * (uint32_t)K + chunk;
    }
    const uint32_t soff = (uint32_t)min(m_start + min((wave & 3) * 64 + lane, W_BM - 1), m_end - 1) * (uint32_t)KT_all * (AS16 ? 2u : 4u);
    // (AS16: 16-bit activation scales staged as they are, see gemm_dma_kernel)
    auto dma_scale = [&](uint32_t lds_addr, int kt_abs) {
        if constexpr (AS16) dma2(lds_addr, soff, (const uint8_t*)p.a_s + (int64_t)kt_abs * 2);
        else dma4(lds_addr, soff, (const uint8_t*)p.a_s + (int64_t)kt_abs * 4);
    };

    // ---- 4-bit weights: a thread owns the same piece of the 128-column half h = 0, 1 of the tile as in the
    // 128-column tile kernel (gemm_dma.hpp): per K step and half one 8-byte load of packed weights and one load
    // of group scales, i.e. four loads per thread and stage like the four weight loads of the other kinds, so
    // that the wait counts of the loop are the same.
    uint32_t w4_off[2] = {0, 0}, w4_soff[2] = {0, 0}, w4_lds[2] = {0, 0};
    if constexpr (W4NK) {
        // thread t: quarter q = t & 3 (16 weights of the 64-element K step) of LDS row (t >> 2) + 128 h
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int Rr = (tid >> 2) + 128 * h, q = tid & 3, rho = Rr & 63;
            const int col = (Rr & 192) + 32 * (rho >> 5) + 8 * ((rho & 15) >> 2) + 4 * ((rho >> 4) & 1) + (rho & 3);
            const uint32_t n = (uint32_t)min(n0 + col, N - 1);
            w4_off[h] = n * (uint32_t)(p.K >> 1) + (uint32_t)q * 8u;               // bytes into the packed matrix
            w4_soff[h] = n * (uint32_t)(p.K / p.group) * 2u;                        // bytes into the scale matrix
            w4_lds[h] = (uint32_t)Rr * 128u + (uint32_t)((2 * q) ^ ((Rr >> 1) & 7)) * 16u;   // chunk 2q; chunk 2q+1 is at ^16
        }
    }
    // (variables of the exact register width, so that no widening move is ever placed between load and wait)
    uint64_t w4_words[2] = {0, 0};
    unsigned w4_scale16[2] = {0, 0};
    auto w4_request = [&](int kt) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if constexpr (W4NK) {
                w4_words[h] = asm_load_b64(w4_off[h], (const uint8_t*)p.b + (int64_t)(kt0 + kt) * 32);
                w4_scale16[h] = asm_load_u16(w4_soff[h], (const uint8_t*)p.b_s + (int64_t)(((kt0 + kt) * 64) / p.group) * 2);
            }
        }
    };
    // the four loads of w4_request(kt) have landed when at most the AL activation loads issued after them are in
    // flight ...
    auto w4_wait = [&]() {
        if constexpr (W4NK)
            asm volatile("s_waitcnt vmcnt(%4)" : "+v"(w4_words[0]), "+v"(w4_scale16[0]), "+v"(w4_words[1]), "+v"(w4_scale16[1]) : "n"(AL) : "memory");
    };
    // ... and, expanded, become the weight rows of stage kt: four pieces (half h = piece >> 1, word piece & 1),
    // which the loop spreads over four MFMA tiles
    auto w4_expand_piece = [&](int kt, int piece) {
        uint8_t* bst = lds + (kt & 1) * W_STAGE + W_A;
        const int h = piece >> 1, jj = piece & 1;
        if constexpr (W4NK) {
            const unsigned s16 = w4_scale16[h];
            const v2h sc = w4_as_h2(s16 | (s16 << 16));
            uint8_t* dst = bst + w4_lds[h];
            if (jj == 0) *(v4i*)dst = w4_word_to_f16x8((unsigned)w4_words[h], sc);
            else *(v4i*)(dst + ((w4_lds[h] & 16u) ? -16 : 16)) = w4_word_to_f16x8((unsigned)(w4_words[h] >> 32), sc);
        }
    };
    auto w4_expand = [&](int kt) {
        w4_wait();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int piece = 0; piece < 4; ++piece) w4_expand_piece(kt, piece);
    };

    // Nothing is in flight when the last K step begins (the step before it ended with vmcnt(0)); this wait costs
    // nothing and puts a covering wait on every static path into that step, also on those that the trip counts
    // rule out (a request in the loop followed by a skipped middle step), which the check of the assembly walks.
    auto w4_drain = [&]() {
        if constexpr (W4NK)
            asm volatile("s_waitcnt vmcnt(0)" : "+v"(w4_words[0]), "+v"(w4_scale16[0]), "+v"(w4_words[1]), "+v"(w4_scale16[1]) : : "memory");
    };

    auto issue = [&](int kt) {
        const uint32_t st = lds_base + (uint32_t)(kt & 1) * W_STAGE;
        const uint8_t* ga = p.a + (int64_t)(kt0 + kt) * 128;
        const uint8_t* gb = bbase + (int64_t)(kt0 + kt) * 128;
        if constexpr (W4) w4_request(kt);          // in front of the activation loads: see w4_expand
#pragma unroll
        for (int i = 0; i < AL; ++i) dma16(st + (uint32_t)(wave * AL + i) * 1024u, aoff[i], ga);
        if constexpr (!W4) {
#pragma unroll
            for (int i = 0; i < 4; ++i) dma16(st + W_A + (uint32_t)(wave * 4 + i) * 1024u, boff[i], gb);
        }
        if constexpr (SCALED) dma_scale(st + W_A + W_B + (uint32_t)(wave & 3) * 256u, kt0 + kt);
    };

    // The loads of a stage inside the loop, a quarter at a time (part 0..3): the weight rows behind the
    // mid-step barrier, the activation rows and the scale column behind the barrier of the step.
    auto issue_part = [&](int kt, int part) {
        const uint32_t st = lds_base + (uint32_t)(kt & 1) * W_STAGE;
        const uint8_t* ga = p.a + (int64_t)(kt0 + kt) * 128;
        if (part < AL) dma16(st + (uint32_t)(wave * AL + part) * 1024u, aoff[part < AL ? part : 0], ga);
        if constexpr (SCALED) if (part == 3) dma_scale(st + W_A + W_B + (uint32_t)(wave & 3) * 256u, kt0 + kt);
    };
    auto issue_b_part = [&](int kt, int part) {
        const uint32_t st = lds_base + (uint32_t)(kt & 1) * W_STAGE;
        dma16(st + W_A + (uint32_t)(wave * 4 + part) * 1024u, boff[part], bbase + (int64_t)(kt0 + kt) * 128);
    };

    // acc[i][j][q] = C[row 16i + r][col 32*(j >> 1) + 8g + 4*(j & 1) + q] of the wave's 16 R x 64 tile
    v4f acc[R][4];
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

    if (KT > 0) issue(0);
    if constexpr (W4) if (KT > 0) w4_expand(0);
    if constexpr (SCALED) {
        for (int i = tid; i < 2 * KT; i += W_THREADS) {
            const int c = i >= KT ? 1 : 0, kk = i - c * KT;
            const int64_t blk = SWIGLU ? (c ? (I_half >> 7) + bx : bx) : min(bx * 2 + c, nblk - 1);
            bsl[c * D_MAX_KT + kk] = ld_scale(p.b_s, bs_off + blk * KT_all + kt0 + kk, p.s_dtype);
        }
    }
    __builtin_amdgcn_s_waitcnt(LLMK_WAIT_VMCNT_0);
    __syncthreads();

    // fragment read offsets inside a 16-row slab: lane group g takes 16-byte chunks g and g + 4 of row r
    // (swizzled).  Both operands use the same K order, so the products are unchanged; with this order the
    // four lane groups of a b128 read hit disjoint bank sets.
    const int lo = r * 128 + ((g ^ ((r >> 1) & 7)) * 16);
    const int hi = r * 128 + (((g + 4) ^ ((r >> 1) & 7)) * 16);
    auto ldfrag = [&](const uint8_t* base) {
        const v4i x = *(const v4i*)(base + lo), y = *(const v4i*)(base + hi);
        return (v8i){x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]};
    };
    // Partial products of a tile row live in one of two register sets: while the MFMAs of row i fill
    // set i & 1, the FMAs scale and accumulate row i - 1 from the other set, four MFMAs after it was
    // produced.  Row 7 of a step is retired by row 0 of the next one, with the scale of its own step.
    v4f t[2][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) t[0][j] = t[1][j] = (v4f){0.f, 0.f, 0.f, 0.f};
    float sprev = 0.f;

    // Fragments of the step being multiplied.  bf and af[0] of step kt + 1 are fetched during the last
    // tile row of step kt, so that a step starts with its operands already in registers.
    v8i bf[4], af[2];
    auto stage_a = [&](int kt) { return lds + (kt & 1) * W_STAGE + (wm * 16 * R) * 128; };
    auto stage_b = [&](int kt) { return lds + (kt & 1) * W_STAGE + W_A + (wn * 64) * 128; };

    // every lane writes two runs of 8 consecutive outputs of each of its rows; row i of the wave tile:
    const int esz = p.c_dtype == LLMK_F32 ? 4 : 2;
    const bool vec_ok = ((((uintptr_t)p.c) & 15) == 0) && (((int64_t)N * esz) % 16 == 0);
    auto store_row = [&](int i) {
        if constexpr (SWIGLU) return;        // nothing is stored before the epilogue below
        const int m = m_start + wm * 16 * R + 16 * i + r;
        if (m >= m_end) return;
        if constexpr (KIND != K_I8_ROWCOL) {
            if (part) {          // work item of a split last round: the fp32 sums of its K range, [tile row][tile column]
                float* dst = part + (wm * 16 * R + 16 * i + r) * W_BN + wn * 64 + 8 * g;
                *(v4f*)dst = acc[i][0];
                *(v4f*)(dst + 4) = acc[i][1];
                *(v4f*)(dst + 32) = acc[i][2];
                *(v4f*)(dst + 36) = acc[i][3];
                return;
            }
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int nbh = n0 + wn * 64 + 32 * h + 8 * g;
            const int nv = N - nbh;
            if (nv <= 0) continue;
            const int64_t off = (int64_t)m * N + nbh;
            if constexpr (KIND == K_I8_ROWCOL) {
                rowcol_epilogue8(p, acc[i][2 * h], acc[i][2 * h + 1], m, off, nbh, nv);
                if (!p.c) continue;
            }
            if (p.c_dtype == LLMK_BF16) store_run8<LLMK_BF16>(p.c, off, acc[i][2 * h], acc[i][2 * h + 1], nv, vec_ok);
            else if (p.c_dtype == LLMK_F16) store_run8<LLMK_F16>(p.c, off, acc[i][2 * h], acc[i][2 * h + 1], nv, vec_ok);
            else store_run8<LLMK_F32>(p.c, off, acc[i][2 * h], acc[i][2 * h + 1], nv, vec_ok);
        }
    };

    // One K step.  SYNC: another step follows; before the last tile row the wave waits for its share of
    // the next stage and for its own LDS reads, and meets the others at the barrier.  Behind the barrier
    // the next stage is complete and nobody reads the current one any more, so the loads of step kt + 2
    // (ISSUE) may overwrite it, and the fragments of step kt + 1 are fetched while the last row is multiplied.
    // NR = tile rows (of 16) this wave multiplies.  Dense GEMM: always R.  Grouped GEMM: the last m-tile of
    // a segment is ragged, and a wave whose rows lie (partly) behind the segment end runs a variant of the
    // loop that neither fetches nor multiplies the tile rows from NR on (their accumulators are never
    // stored); the loop is instantiated for NR = R, R / 2 and 0 so that it stays free of branches (a two-row variant
    // measured no faster: short tails are bound by the per-step barrier, not by the matrix pipe).
    auto step = [&](int kt, auto sync_c, auto issue_c, auto nr_c) {
        constexpr bool SYNC = decltype(sync_c)::value, ISSUE = decltype(issue_c)::value;
        constexpr int NR = decltype(nr_c)::value;
        if constexpr (W4 && !SYNC) w4_drain();
        const uint8_t* As = stage_a(kt);
        float sa[R];
        if constexpr (SCALED && NR > 0) {
            const float* Ss = (const float*)(lds + (kt & 1) * W_STAGE + W_A + W_B) + wm * 16 * R + r;
            const float bs = bsl[(wn >> 1) * D_MAX_KT + kt];
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                if constexpr (AS16) {
                    const unsigned raw = ((const unsigned*)Ss)[i * 16];
                    sa[i] = (p.s_dtype == LLMK_F16 ? f16_to_f32((unsigned short)raw) : bf16_to_f32((unsigned short)raw)) * bs;
                } else {
                    sa[i] = Ss[i * 16] * bs;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < R; ++i) {
            if (i + 1 < NR) af[(i + 1) & 1] = ldfrag(As + (i + 1) * 2048);
            if constexpr (W4) {
                // 4-bit weights: the packed words of step kt + 1, requested a step ago, become the weight rows of
                // the other stage (nobody has read those since the barrier of step kt - 1, so no barrier here),
                // and the words of step kt + 2 are requested into the registers just freed.
                if (i == W_EARLY_ROW && SYNC) {
                    __builtin_amdgcn_sched_barrier(0);
                    w4_wait();
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else if (i == W_EARLY_ROW && ISSUE) {
                // Every wave has had its weight fragments of this step in registers since the step began, so
                // behind this barrier the weight half of the stage may be overwritten: the weight loads of
                // step kt + 2 go out here, the activation loads behind the barrier of row 7.  Two bursts of
                // loads per step instead of one measured 4-6 % faster (rows 4 and 5 best, 0 and 1 no gain).
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
            }
            if (i == R - 1 && SYNC) {
                __builtin_amdgcn_sched_barrier(0);
                // vmcnt(4): the four weight loads of step kt + 2 may stay in flight; lgkmcnt(0)
                if constexpr (ISSUE) __builtin_amdgcn_s_waitcnt(0x0074);
                else __builtin_amdgcn_s_waitcnt(0x0070);
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if constexpr (SCALED) {
                    if (i < NR) t[i & 1][j] = step_dot<KIND>(bf[j], af[i & 1]);
                    if (i > 0 && i <= NR) acc[i - 1][j] += t[(i - 1) & 1][j] * sa[i - 1];
                    else if (i == 0 && NR == R) acc[R - 1][j] += t[1][j] * sprev;
                } else {
                    if (i < NR) acc[i][j] = mma_plain<KIND>(bf[j], af[i & 1], acc[i][j]);
                }
                if constexpr (W4) {
                    if (i == W_EARLY_ROW && SYNC) {
                        w4_expand_piece(kt + 1, j);
                        if (j == 3 && ISSUE) w4_request(kt + 2);
                    }
                } else if (i == W_EARLY_ROW && ISSUE) issue_b_part(kt + 2, j);
                if (i == R - 1 && SYNC) {
                    if (ISSUE) issue_part(kt + 2, j);      // a quarter behind each tile (0.5-1 % faster than all at once)
                    if (NR > 0) {
                        bf[j] = ldfrag(stage_b(kt + 1) + j * 2048);
                        if (j == 3) af[0] = ldfrag(stage_a(kt + 1));
                    }
                }
                // Nothing moves across a tile boundary: the FMAs retire a product finished four MFMAs
                // ago, never the one just issued, and each activation fragment is requested a whole
                // tile row before its first use.
                __builtin_amdgcn_sched_barrier(0);
            }
            // last K step: the outputs of tile row i - 1 are final once row i has been issued; storing them
            // here overlaps the conversion and the write with the rest of the step
            if constexpr (!SYNC) {
                if (i >= 1 && i <= NR) store_row(i - 1);
            }
        }
        if constexpr (SCALED && NR == R) sprev = sa[R - 1];
    };

    if (KT > 1) issue(1);
    if (KT > 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) bf[j] = ldfrag(stage_b(0) + j * 2048);
        af[0] = ldfrag(stage_a(0));
    }
    const std::true_type yes;
    const std::false_type no;
    auto run = [&](auto nr_c) {
        int kt = 0;
        for (; kt + 2 < KT; ++kt) step(kt, yes, yes, nr_c);
        if (kt + 1 < KT) { step(kt, yes, no, nr_c); ++kt; }
        if (kt < KT) step(kt, no, no, nr_c);
        if constexpr (SCALED && decltype(nr_c)::value == R) {
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[R - 1][j] += t[1][j] * sprev;
        }
    };
    if constexpr (GROUPED) {
        const int live = m_end - m_start - wm * 16 * R;    // rows of this wave inside the segment (wave-uniform)
        if (live > 8 * R) run(std::integral_constant<int, R>{});
        else if (live > 0) run(std::integral_constant<int, R / 2>{});
        else run(std::integral_constant<int, 0>{});
    } else {
        run(std::integral_constant<int, R>{});
    }

    if constexpr (SWIGLU) {
        // ---- gated activation + 1 x 128 quantiser.  Waves wn = 0, 1 hold the gate columns of the wave's 16 R rows, waves
        // wn = 2, 3 the up columns of the same rows, same lane and register for the same (row, column).  The pair (wn,
        // wn + 2) splits the rows: the gate wave finishes tile rows 0 .. R/2 - 1, the up wave rows R/2 .. R - 1, after each
        // has passed the other its half through LDS (16-bit values, as the GEMM would have stored them).  A group of
        // 128 outputs of a row lies in two waves (wn & 1), whose row maxima meet in LDS.
        constexpr int RH = R / 2;
        constexpr bool FP8Q = (KIND == K_FP8_BLOCK);
        uint8_t* const xch = lds;                                        // [wave][RH][2][64 lanes] x 16 bytes
        float* const rowmax = (float*)(lds + 8 * RH * 2 * 1024);         // [wm][half][wn & 1][16 RH rows]
        const int half = wn >> 1, w1 = wn & 1;
        const int gcols = I_half >> 7;                                   // scale groups per output row
        auto pack8 = [&](const v4f& x, const v4f& y) {
            v4i w;
            if (p.c_dtype == LLMK_F16) {
                w[0] = (int)pack_f16x2(x[0], x[1]); w[1] = (int)pack_f16x2(x[2], x[3]);
                w[2] = (int)pack_f16x2(y[0], y[1]); w[3] = (int)pack_f16x2(y[2], y[3]);
            } else {
                w[0] = (int)pack_bf16x2(x[0], x[1]); w[1] = (int)pack_bf16x2(x[2], x[3]);
                w[2] = (int)pack_bf16x2(y[0], y[1]); w[3] = (int)pack_bf16x2(y[2], y[3]);
            }
            return w;
        };
        auto epilogue = [&](auto half_c, auto idt_c) {
            constexpr int HALF = decltype(half_c)::value, IDT = decltype(idt_c)::value;
            constexpr int OWN = RH * HALF, OTH = RH * (1 - HALF);
            __syncthreads();                                             // every wave is done with the stages
            {
                uint8_t* dst = xch + (uint32_t)(wave * RH * 2) * 1024u + (uint32_t)lane * 16u;
#pragma unroll
                for (int i = 0; i < RH; ++i)
#pragma unroll
                    for (int h = 0; h < 2; ++h) *(v4i*)(dst + (i * 2 + h) * 1024) = pack8(acc[OTH + i][2 * h], acc[OTH + i][2 * h + 1]);
            }
            __syncthreads();
            // partner: same wm and wn & 1, other half
            const int partner = wm * 4 + (1 - HALF) * 2 + w1;
            const uint8_t* src = xch + (uint32_t)(partner * RH * 2) * 1024u + (uint32_t)lane * 16u;
            float y[RH][2][EPL], mx[RH];
#pragma unroll
            for (int i = 0; i < RH; ++i) {
                float m = 0.f;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    float other[EPL], own[EPL];
                    const v4i wo = *(const v4i*)(src + (i * 2 + h) * 1024);
                    const v4i wm_ = pack8(acc[OWN + i][2 * h], acc[OWN + i][2 * h + 1]);
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const unsigned a = (unsigned)wo[q], b = (unsigned)wm_[q];
                        if constexpr (IDT == LLMK_F16) {
                            other[2 * q] = f16_to_f32((unsigned short)a); other[2 * q + 1] = f16_to_f32((unsigned short)(a >> 16));
                            own[2 * q] = f16_to_f32((unsigned short)b); own[2 * q + 1] = f16_to_f32((unsigned short)(b >> 16));
                        } else {
                            other[2 * q] = bf16_to_f32((unsigned short)a); other[2 * q + 1] = bf16_to_f32((unsigned short)(a >> 16));
                            own[2 * q] = bf16_to_f32((unsigned short)b); own[2 * q + 1] = bf16_to_f32((unsigned short)(b >> 16));
                        }
                    }
#pragma unroll
                    for (int q = 0; q < EPL; ++q) {
                        const float gv = HALF == 0 ? own[q] : other[q], up = HALF == 0 ? other[q] : own[q];
                        y[i][h][q] = gated_act<IDT>(gv, up, p.act, false, 1.0f);
                        m = fmaxf(m, fabsf(y[i][h][q]));
                    }
                }
                m = fmaxf(m, __shfl_xor(m, 16, 64));
                m = fmaxf(m, __shfl_xor(m, 32, 64));
                mx[i] = m;
                if (g == 0) rowmax[((wm * 2 + HALF) * 2 + w1) * (16 * RH) + 16 * i + r] = m;
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < RH; ++i) {
                const float m = fmaxf(mx[i], rowmax[((wm * 2 + HALF) * 2 + (1 - w1)) * (16 * RH) + 16 * i + r]);
                const int row = m_start + wm * 16 * R + 16 * (OWN + i) + r;
                if (row >= m_end) continue;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int col = n0 + 64 * w1 + 32 * h + 8 * g;
                    quant_store8<FP8Q>(y[i][h], m, p.c, (int64_t)row * I_half + col, p.q_scale, (int64_t)row * gcols + bx,
                                       w1 == 0 && g == 0 && h == 0, p.round_mode);
                }
            }
        };
        const std::integral_constant<int, 0> h0;
        const std::integral_constant<int, 1> h1;
        const std::integral_constant<int, LLMK_F16> tf16;
        const std::integral_constant<int, LLMK_BF16> tbf16;
        if (p.c_dtype == LLMK_F16) { if (half == 0) epilogue(h0, tf16); else epilogue(h1, tf16); }
        else { if (half == 0) epilogue(h0, tbf16); else epilogue(h1, tbf16); }
        return;
    }

    // ---- epilogue: the rows not yet stored by the last K step
    if (KT > 0) store_row(R - 1);
    else {
#pragma unroll
        for (int i = 0; i < R; ++i) store_row(i);
    }
    if (clocked) {
        p.clocks[0] = clock64() - clk0;
        p.clocks[1] = wall_clock64() - wall0;
    }
}

// Adds the partial sums of the split last round (see wide_tail_plan) and writes the outputs of its tiles: grid
// (tiles of that round, slices of 32 tile rows), the K ranges in ascending order (the result does not depend on
// timing); a thread sums eight rows at a time so that eight loads are in flight per K range.
template <bool GROUPED, int R>
__global__ __launch_bounds__(256) void wide_tail_sum_kernel(DirectArgs p, int esz) {
    constexpr int W_BM = w_bm(R);
    const int gx = (p.N + W_BN - 1) / W_BN;
    const WideTail tp = wide_tail_plan(wide_total_tiles<GROUPED, R>(p, gx), (p.K * esz) >> 7);
    const int idx = blockIdx.x;
    if (tp.z <= 1 || idx >= tp.ntail) return;
    const WideTile wt = wide_tile_of<GROUPED, R>(p, tp.full + idx, gx);
    if (!wt.found) return;
    const int rows = wt.m_end - wt.m_start, c4 = (threadIdx.x & 63) * 4, n = wt.bx * W_BN + c4;
    const int row0 = (int)blockIdx.y * 32 + (threadIdx.x >> 6);
    if ((int)blockIdx.y * 32 >= rows) return;
    v4f s[8];
#pragma unroll
    for (int it = 0; it < 8; ++it) s[it] = (v4f){0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < tp.z; ++k) {
        const float* src = p.partial + ((int64_t)(k * tp.ntail + idx) * W_BM + row0) * W_BN + c4;
#pragma unroll
        for (int it = 0; it < 8; ++it) s[it] += *(const v4f*)(src + it * 4 * W_BN);      // rows past the tile end: stale scratch, not stored
    }
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int row = row0 + 4 * it;
        if (row >= rows) continue;
        const int64_t off = (int64_t)(wt.m_start + row) * p.N + n;
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (n + q < p.N) st_out(p.c, off + q, s[it][q], p.c_dtype);
    }
}

// scratch of the split last round: W_TAIL_ITEMS partial tiles of the larger tile shape
constexpr int64_t w_tail_bytes() { return (int64_t)W_TAIL_ITEMS * w_bm(8) * W_BN * 4; }

template <int KIND, bool GROUPED, int R = 8>
int launch_wide(const DirectArgs& p0, hipStream_t stream, const char* name, void* ws = nullptr, int64_t ws_bytes = 0) {
    static std::atomic<uint64_t> configured{0};
    auto kern = gemm_wide_kernel<KIND, GROUPED, R>;
    constexpr int W_BM = w_bm(R), W_LDS = w_lds(R);
    constexpr int ESZ = (KIND == K_F16 || KIND == K_BF16 || KIND == K_W4NK) ? 2 : 1;
    if (int rc = llmk_reserve_lds((const void*)kern, W_LDS, configured, name)) return rc;
    DirectArgs p = p0;
    const int tiles_m = GROUPED ? grouped_row_tiles(p.M, p.E, W_BM) : (p.M + W_BM - 1) / W_BM;
    dim3 grid((unsigned)((p.N + W_BN - 1) / W_BN), (unsigned)tiles_m);
    if (grid.x == 0 || grid.y == 0) return LLMK_OK;
    // a short last round of tiles is split along K when the scratch for its partial sums is there (dense: decided
    // here; grouped: the segment ends are known on the device only, so the kernel decides, from 256 tiles on)
    bool tail = false;
    p.tail_split = 0;
    if constexpr (KIND == K_FP8_BLOCK || KIND == K_I8_BLOCK || KIND == K_F16 || KIND == K_BF16) {
        const int KT = (p.K * ESZ) >> 7;
        // (the split is planned for rounds of LLMK_CUS workgroups: taken only on a device with that many CUs)
        if (ws && ws_bytes >= w_tail_bytes() && !((uintptr_t)ws & 15) && KT >= W_TAIL_MIN_KT && p.c && llmk_device_cus() == LLMK_CUS)
            tail = GROUPED ? (int64_t)grid.x * grid.y >= LLMK_CUS : wide_tail_plan((int)(grid.x * grid.y), KT).z > 1;
    }
    if (tail) {
        p.tail_split = 1;
        p.partial = (float*)ws;
        grid.y += (W_TAIL_ITEMS + grid.x - 1) / grid.x;     // the work items of the split round
    }
    kern<<<grid, W_THREADS, W_LDS, stream>>>(p);
    LLMK_CHECK_LAUNCH(name);
    if (tail) {
        wide_tail_sum_kernel<GROUPED, R><<<dim3(LLMK_CUS / 2, W_BM / 32), 256, 0, stream>>>(p, ESZ);
        LLMK_CHECK_LAUNCH(name);
    }
    return LLMK_OK;
}

// The gated-activation form of the kernel (grouped gate / up projection, p.N = 2 I, I % 128 == 0): one column tile per
// 128 gate columns; no split of the last round (its tiles would have to meet before the activation).
template <int KIND, int R>
int launch_wide_swiglu(const DirectArgs& p, hipStream_t stream, const char* name) {
    static std::atomic<uint64_t> configured{0};
    auto kern = gemm_wide_kernel<KIND, true, R, true>;
    constexpr int W_BM = w_bm(R), W_LDS = w_lds(R);
    static_assert(8 * (R / 2) * 2 * 1024 + 2 * 2 * 2 * 16 * (R / 2) * 4 <= W_LDS, "exchange area and row maxima fit in the stages");
    if (int rc = llmk_reserve_lds((const void*)kern, W_LDS, configured, name)) return rc;
    dim3 grid((unsigned)((p.N / 2) / 128), (unsigned)grouped_row_tiles(p.M, p.E, W_BM));
    if (grid.x == 0 || grid.y == 0) return LLMK_OK;
    kern<<<grid, W_THREADS, W_LDS, stream>>>(p);
    LLMK_CHECK_LAUNCH(name);
    return LLMK_OK;
}

// K split of the 64-row-tile kernel: as many slices as bring the grid to about one workgroup per CU, each
// slice at least eight K steps long; 1 = no split.  (Also sizes the scratch, so it depends on the shape only.)
// With 128 or more tiles the summing pass costs what two slices save unless K is long.
inline int splitk_factor(int64_t M, int64_t N, int64_t K) {
    if (M <= 16 || M > 512) return 1;
    const int64_t tiles = ((M + 63) / 64) * ((N + 127) / 128);
    if (tiles >= LLMK_CUS || (tiles >= LLMK_CUS / 2 && K < 8192)) return 1;
    int64_t z = (LLMK_CUS - 1 + tiles) / tiles;
    z = z < (K >> 10) ? z : (K >> 10);
    return (int)(z > 8 ? 8 : (z < 1 ? 1 : z));
}

// Shapes for the mid-size kernel (gemm_mid.hpp): more than 64 rows, at most one workgroup per CU and a K range of at
// most 8 KB per row, 16 KB on the 64-row tile.  Measured against the 128-column tile kernels (fp8, us per launch, cold
// weights): 128 x 4096 x 4096 16.7 -> 12.7, 256 x 4096 x 4096 23.1 -> 15.3, 256 x 4096 x 8192 28.7 -> 24.2,
// 256 x 4096 x 14336 44.2 -> 39.0 (K slices of the 64 x 128 tile before); with more than one round of workgroups, or on
// the 32-row tile with rows beyond 8 KB, it loses (512 x 4096 x 4096 15.5 -> 23.4, 256 x 6144 x 4096 23.5 -> 27.9,
// 128 x 4096 x 14336 28.4 -> 29.2, per-token int8 26.2 -> 30.4).
inline bool mid_wanted(int64_t M, int64_t N, int64_t kbytes) {
    if (M <= 64 || M > 512) return false;
    const MidPlan pl = mid_plan(M, N, kbytes);
    return pl.tiles <= LLMK_CUS && kbytes <= (pl.mt == 4 ? 16384 : 8192);
}

// Shapes for the 128-column form of that kernel: shapes the 64-column form does not take, one round of 64- or 128-row
// tiles, rows of at most 16 KB (256 x 14336 x 14336 118.4 -> 86.3 us, 128 x 14336 x 14336 85.4 -> 65.7, 128 x 4096 x 14336
// in four K slices 28.4 -> 27.0).  Taken for fp8 and for fp16 activations with row-packed 4-bit weights, where it beats
// the 128-column tile kernels (fp8, us per launch, cold weights: 128 x 14336 x 4096 26.3 -> 23.2, 256 x 14336 x 4096
// 37.6 -> 29.6, 256 x 6144 x 4096 23.6 -> 20.2, 128 x 28672 x 4096 44.3 -> 38.6, 384 x 8192 x 4096 35.1 -> 27.7,
// 128 x 14336 x 8192 53.5 -> 38.9; 4-bit 128 x 14336 x 4096 37.1 -> 33.2, same elsewhere); the int8 kinds lose on it
// (per-token 128 x 14336 x 4096 23.9 -> 25.9, 256 x 14336 x 4096 28.9 -> 34.7; block-scaled 34.8 -> 37.4) and stay where
// they were, and two rounds of its workgroups lose everywhere (fp8 256 x 28672 x 4096 48.6 -> 62.6).
inline bool midw_wanted(int64_t M, int64_t N, int64_t kbytes) {
    if (M <= 64 || M > 512 || kbytes > 16384) return false;
    return midw_plan(M, N, kbytes).tiles <= LLMK_CUS;
}

// 16 < M <= 64: the weight-streaming kernel re-reads the activations for every 16 columns, which costs more
// than the 64-row tile kernel (with split-K when its tiles are few) once the weight matrix is large (measured
// crossover between 17 M and 25 M elements).
inline bool mid_m_prefers_tiles(int64_t M, int64_t N, int64_t K) {
    return M > 16 && M <= 64 && N * K >= (int64_t)20 << 20;
}

// Tile shape by estimated time: rounds of 256 workgroups times the measured cost of one round of each tile
// shape (60 / 36 / 43 / 26 / 16 microseconds for 256 x 256, 128 x 256, 256 x 128, 128 x 128 and 64 x 128 at K = 4096
// for fp8; the ratios hold for the other kinds and K).  Ties go to the larger tile (less operand re-reading).  Segments of a grouped GEMM are judged by their average length.
// which tile shape the estimate picks: 8 / 9 = the 256 x 256 / 128 x 256 tile of gemm_wide_kernel, 4 / 2 / 1 = MI of gemm_dma_kernel
template <int KIND, bool GROUPED>
int dma_tile_choice(const DirectArgs& p) {
    // 4-bit weights: the row-packed layout, dense launches (the Marlin scatter of 2-byte pieces measured 4-9 % slower
    // inside the 256-column kernel than the dequantisation pass at every M > 512)
    constexpr bool HAS_WIDE = KIND != K_W4MARLIN && KIND != K_W4A8 && !(GROUPED && KIND == K_W4NK);
    const int64_t rows = GROUPED ? p.M / (p.E > 0 ? p.E : 1) : p.M;
    const int64_t groups = GROUPED ? p.E : 1;
    // a segment of a grouped GEMM rarely ends on a tile boundary: count one ragged tile per segment on top of
    // the full ones (with the plain ceiling, segments of 128 +- a few rows looked like one 128-row tile each and
    // went to a tile shape that needed two; -8 % on the Mixtral forward at 256 and 512 tokens)
    auto rounds = [&](int bm, int bn) { return (((p.N + bn - 1) / bn) * groups * (GROUPED ? rows / bm + 1 : (rows + bm - 1) / bm) + LLMK_CUS - 1) / LLMK_CUS; };
    const double t_wide = 60.0 * rounds(256, 256), t4 = 43.0 * rounds(256, 128), t2 = 26.0 * rounds(128, 128),
                 t1 = 16.0 * rounds(64, 128);
    if constexpr (HAS_WIDE) {
        if (t_wide <= t4 && t_wide <= t2 && t_wide <= t1) {
            // problems whose 256 x 256 tiles do not fill a round: the 128 x 256 tile of the same kernel
            // (a tie goes to the 128-row tile for block-scaled int8, whose per-step conversions leave the tall
            // tile less of its advantage: grouped Mixtral down projection -3 %; +1 % for fp8)
            const double t_half = 36.0 * rounds(128, 256);
            if (t_half < t_wide || (KIND == K_I8_BLOCK && GROUPED && t_half == t_wide)) return 9;
            return 8;
        }
        const double t_half = 36.0 * rounds(128, 256);
        if (t_half < t4 && t_half <= t2 && t_half <= t1) return 9;
    }
    int max_mi = 4;
    if constexpr (KIND == K_W4A8) max_mi = w4a8_max_mi(p);       // the table of zero points and scales must fit behind the stages
    if constexpr (KIND != K_W4A8) {
        if (t4 <= t2 && t4 <= t1 && max_mi >= 4) return 4;
    }
    if (t2 <= t1 && max_mi >= 2) return 2;
    return 1;
}

// AS16 (16-bit activation scales staged as they are): the 64- and 128-row tiles of gemm_dma_kernel only, see launch_big
template <int KIND, bool GROUPED, bool AS16 = false>
int launch_dma(const DirectArgs& p, hipStream_t stream, const char* name, void* ws = nullptr, int64_t ws_bytes = 0) {
    if (!GROUPED && p.ksplit > 1) return launch_dma_mi<KIND, GROUPED, 1, AS16>(p, stream, name);
    const int choice = dma_tile_choice<KIND, GROUPED>(p);
    if constexpr (!AS16) {
        if constexpr (KIND != K_W4MARLIN && KIND != K_W4A8 && !(GROUPED && KIND == K_W4NK)) {
            if (choice == 9) return launch_wide<KIND, GROUPED, 4>(p, stream, name, ws, ws_bytes);
            if (choice == 8) return launch_wide<KIND, GROUPED, 8>(p, stream, name, ws, ws_bytes);
        }
        if constexpr (KIND != K_W4A8) {
            if (choice == 4) return launch_dma_mi<KIND, GROUPED, 4>(p, stream, name);
        }
    }
    if (choice == 2) return launch_dma_mi<KIND, GROUPED, 2, AS16>(p, stream, name);
    return launch_dma_mi<KIND, GROUPED, 1, AS16>(p, stream, name);
}

// Dispatch for the compute-bound block-scaled GEMM: direct-to-LDS kernels when eligible (converting
// 16-bit activation scales into `workspace` first), register-staged two-stage kernel otherwise.
template <int KIND, bool GROUPED>
int launch_big(DirectArgs p, void* workspace, int64_t workspace_bytes, hipStream_t stream, const char* name) {
    if (!dma_eligible(p)) return launch_tiled<KIND, GROUPED>(p, stream, name);
    // Mid-size M on few column tiles: the 64-column kernel with 512-byte K steps; it stages 16-bit activation scales
    // as they are, so no widening pass runs in front of it
    if constexpr (!GROUPED) {
        if (mid_wanted(p.M, p.N, p.K) && (KIND != K_FP8_BLOCK || p.s_dtype == LLMK_F32)) {
            MidPlan pl = mid_plan(p.M, p.N, p.K);
            const int64_t need = (int64_t)pl.z * p.M * p.N * 4;
            if (pl.z > 1 && !(workspace && workspace_bytes >= need && !(((uintptr_t)workspace) & 15))) pl.z = 1;
            if (mid_eligible<KIND>(p, pl.mt, pl.z)) {
                if (pl.z > 1) { p.partial = (float*)workspace; p.ksplit = pl.z; }
                if (p.s_dtype != LLMK_F32) {
                    if constexpr (KIND != K_FP8_BLOCK)
                        return pl.mt == 4 ? launch_mid<KIND, 4, true>(p, stream, name) : launch_mid<KIND, 2, true>(p, stream, name);
                }
                return pl.mt == 4 ? launch_mid<KIND, 4>(p, stream, name) : launch_mid<KIND, 2>(p, stream, name);
            }
        }
    }
    if constexpr (!GROUPED) {
        // wider weights: the 128-column form of the same kernel (fp8; see midw_wanted)
        if (KIND == K_FP8_BLOCK && p.s_dtype == LLMK_F32 && midw_wanted(p.M, p.N, p.K)) {
            MidPlan pl = midw_plan(p.M, p.N, p.K);
            const int64_t need = (int64_t)pl.z * p.M * p.N * 4;
            if (pl.z > 1 && !(workspace && workspace_bytes >= need && !(((uintptr_t)workspace) & 15))) pl.z = 1;
            if (dma_eligible(p)) {
                if (pl.z > 1) { p.partial = (float*)workspace; p.ksplit = pl.z; }
                if constexpr (KIND == K_FP8_BLOCK)
                    return pl.mt == 4 ? launch_mid<KIND, 4, false, true>(p, stream, name) : launch_mid<KIND, 8, false, true>(p, stream, name);
            }
        }
    }
    int64_t used = 0;
    // 16-bit activation scales: the int8 kind stages them as they are (AS16 instantiations); fp8 callers pass fp32
    // scales as a rule, 16-bit ones are widened into the workspace first
    constexpr bool HAS_AS16 = (KIND == K_I8_BLOCK);
    // (only where the launch is short: the conversion inside the K loop costs the vector-ALU-bound int8 loop 4-5 %,
    // the widening pass a launch of 5-7 us: 512 x 4096 x 4096 21.4 -> 17.8 us, 1024 x 4096 x 4096 28.0 -> 26.5 us, but
    // 4096 x 14336 x 4096 277.6 -> 291 us when forced; the 64- and 128-row tiles are the short launches)
    bool as16 = false;
    if constexpr (HAS_AS16) {
        if (p.s_dtype != LLMK_F32) {
            const int z = GROUPED ? 1 : splitk_factor(p.M, p.N, p.K);
            as16 = z > 1 || dma_tile_choice<KIND, GROUPED>(p) <= 2;
        }
    }
    if (p.s_dtype != LLMK_F32 && !as16) {
        const int64_t n = (int64_t)p.M * (p.K >> 7);
        if (!workspace || workspace_bytes < n * 4) return launch_tiled<KIND, GROUPED>(p, stream, name);
        const unsigned blocks = (unsigned)cdiv64(n, 256);
        if (p.s_dtype == LLMK_F16) scales_to_f32_kernel<LLMK_F16><<<blocks, 256, 0, stream>>>(p.a_s, (float*)workspace, n);
        else scales_to_f32_kernel<LLMK_BF16><<<blocks, 256, 0, stream>>>(p.a_s, (float*)workspace, n);
        LLMK_CHECK_LAUNCH(name);
        p.a_s = workspace;
        used = (n * 4 + 255) & ~(int64_t)255;
    }
    // Few 64-row tiles (mid-size M, moderate N): split K over workgroups so that every CU streams weights,
    // fp32 partials in the workspace, one summing pass.
    if constexpr (!GROUPED) {
        const int z = splitk_factor(p.M, p.N, p.K);
        const int64_t need = (int64_t)z * p.M * p.N * 4;
        if (z > 1 && workspace && workspace_bytes - used >= need && !(((uintptr_t)workspace + used) & 15)) {
            p.partial = (float*)((uint8_t*)workspace + used);
            p.ksplit = z;
        }
    }
    if constexpr (HAS_AS16) {
        if (as16) {
            if (p.ksplit > 1 || !workspace) return launch_dma<KIND, GROUPED, true>(p, stream, name);
            return launch_dma<KIND, GROUPED, true>(p, stream, name, workspace, workspace_bytes);                  // split last round
        }
    }
    if (p.ksplit > 1 || !workspace || workspace_bytes <= used) return launch_dma<KIND, GROUPED>(p, stream, name);
    return launch_dma<KIND, GROUPED>(p, stream, name, (uint8_t*)workspace + used, workspace_bytes - used);   // split last round
}

// K slices for the half-precision tile kernel (a K step is 64 elements there): same rule as splitk_factor
inline int splitk_factor_half(int64_t M, int64_t N, int64_t K) { return splitk_factor(M, N, 2 * K); }

// fp16 / bf16 operands, no scales (K % 64 == 0); `workspace` (optional) holds the fp32 split-K partials
template <int KIND, bool GROUPED>
int launch_big_half(DirectArgs p, hipStream_t stream, const char* name, void* workspace = nullptr, int64_t workspace_bytes = 0) {
    if (!dma_eligible(p, 2)) LLMK_FAIL(LLMK_ERR_SHAPE, "%s: shape not supported by the tiled half-precision kernel", name);
    if constexpr (!GROUPED) {
        int z = splitk_factor_half(p.M, p.N, p.K);
        if constexpr (KIND == K_W4MARLIN) {
            // a round of 64-row tiles costs this kind 44 us at K = 4096 whatever its width (the scatter of the Marlin
            // layout), so the slices must not open a second round: at most 256 / tiles of them (128 x 14336 x 4096:
            // 51.9 us in two slices, 44.0 unsplit; 256 x 6144 x 4096 51.1 -> 43.9; 128 x 8192 x 4096 keeps two: 30.2 vs 43.5)
            const int64_t tiles = (((int64_t)p.M + 63) / 64) * (((int64_t)p.N + 127) / 128);
            const int zmax = (int)(LLMK_CUS / tiles > 1 ? LLMK_CUS / tiles : 1);
            if (z > zmax) z = zmax;
        }
        if (z > 1 && workspace && workspace_bytes >= (int64_t)z * p.M * p.N * 4 && !(((uintptr_t)workspace) & 15)) {
            p.partial = (float*)workspace;
            p.ksplit = z;
        }
    }
    if (p.ksplit > 1) return launch_dma<KIND, GROUPED>(p, stream, name);
    return launch_dma<KIND, GROUPED>(p, stream, name, workspace, workspace_bytes);                             // split last round
}

}  // namespace llmk
