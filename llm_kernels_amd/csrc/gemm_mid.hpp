// Tile kernels for mid-size M (about 65 to 512 rows) on few column tiles: problems that neither fill the chip with
// 128- or 256-column tiles nor fit the weight-streaming kernels, and whose weights mostly come cold from HBM.
//
// What bounds the 64 x 128 tile of gemm_dma.hpp there is the per-step overhead: one barrier, twelve fragment reads
// and a dependent wait per wave for four matrix instructions on 128 bytes of K.  Here a K step is 512 bytes = four
// 128-byte sub-blocks, the tile is 16 MT x 64 (MT = 4 or 2), a wave multiplies ONE sub-block of the step, and the four
// partial sums of an output meet in LDS once, at the end of the tile (a K split inside the workgroup: one barrier per
// 512 bytes of K).  Activations (hot in L2: every workgroup of a row tile reads the same rows) go global -> LDS by
// direct-to-LDS loads one step ahead, two stages.  Weights (cold: each byte is needed by M / (16 MT) workgroups only)
// go global -> registers several steps ahead, coalesced (eight lanes per 128-byte line), by hand-issued loads into a
// ring of register sets, and from there into one of two LDS stages one step before they are multiplied: weight bytes
// in flight without spending LDS on them, and a natural place to unpack 4-bit weights.  The row tiles that share a
// column tile land on one XCD (same workgroup id modulo 8 when the column tiles are a multiple of 8) and walk K in
// step, so that a weight line comes from HBM once.
//
// Two forms:
//   gemm_mid_kernel     (K_W4A8): all eight waves load, unpack and multiply: wave (wn, kq) takes 32 columns of sub-block
//                       kq.  The unpacking (q - z4) * s4 is vector-ALU work that wants every wave.
//   gemm_mid_pc_kernel  (every other kind): four waves only request and stage operands, four only multiply; see there.
//
// All loads of a step are issued unconditionally (steps past the end repeat the last one) so that one
// hand-counted s_waitcnt per step is exact; check_asm.py proves the register loads on every build.
#pragma once
#include "gemm_dma.hpp"

namespace llmk {

constexpr int MD_BN = 64, MD_THREADS = 512;

constexpr int MD_B = 4 * MD_BN * 128;                       // weight stage: [sub-block][column][128 B] = 32 KB
constexpr int MD_S = 4 * 64 * 4;                            // activation-scale columns of a step: [sub-block][row] fp32
constexpr int MD_RED_ROW = 68;                              // floats per row of the final reduction (64 + 4: bank spread)
constexpr int md_a(int mt) { return 4 * 16 * mt * 128; }    // activation stage: [sub-block][row][128 B]
constexpr int MD_NA = 2;                                    // activation stages
constexpr int MD_NBS = 2;                                   // weight stages
constexpr int md_stages(int mt) { return MD_NA * (md_a(mt) + MD_S) + MD_NBS * MD_B; }
constexpr int md_red(int mt) { return 4 * 16 * mt * MD_RED_ROW * 4; }
// stages (reused by the reduction), weight-scale table, K_W4A8 table of zero points and second-level scales
constexpr int md_lds(int mt, int kt_tab) { return md_stages(mt) + D_MAX_KT * 4 + 128 * kt_tab; }

// f(integral_constant<I>) for I = FIRST .. LAST - 1 (ring slots are compile-time indices)
template <int I, int LAST, class F>
__device__ __forceinline__ void md_static_for(F&& f) {
    if constexpr (I < LAST) {
        f(std::integral_constant<int, I>{});
        md_static_for<I + 1, LAST>(f);
    }
}
// the same, nested: f(I) runs only if rem > I and f(I - 1) ran (a later step without the earlier ones is a path the
// trip count rules out, and the static check of the assembly would still walk it)
template <int I, int LAST, class F>
__device__ __forceinline__ void md_static_nested(int rem, F&& f) {
    if constexpr (I < LAST) {
        if (rem > I) {
            f(std::integral_constant<int, I>{});
            md_static_nested<I + 1, LAST>(rem, f);
        }
    }
}

// AS16: the activation scales are 16-bit (fp16 or bf16 by p.s_dtype) and are staged as they are (one zero-extended
// element per dword slot of the scale column) instead of being widened to fp32 by a kernel of their own first.
template <int KIND, int MT, bool AS16 = false>
__global__ __launch_bounds__(MD_THREADS) void gemm_mid_kernel(DirectArgs p) {
    static_assert(MT == 4 || MT == 2, "tile rows");
    static_assert(KIND == K_W4A8, "the other kinds run on gemm_mid_pc_kernel");
    constexpr int BM = 16 * MT;
    constexpr int MD_A = md_a(MT);
    constexpr int NB = 2;                                   // ring loads per thread and step
    constexpr int MD_RING = 4;                              // ring slots: weights are requested MD_RING - 1 steps ahead
    constexpr int NA = MT + 1;                              // direct-to-LDS loads per thread and step (activation pieces, scale column)
    static_assert(md_red(MT) <= md_stages(MT), "the reduction reuses the stages");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4, wn = wave & 1, kq = wave >> 1;
    const int N = p.N;
    const int K = p.K;                                      // row length in bytes (int8 activations)
    const int KT_all = K >> 7;                              // 128-byte sub-blocks per row
    int kt0 = 0, KT = KT_all;                               // sub-blocks [kt0, kt0 + KT) of this workgroup
    if (p.ksplit > 1) {
        // slices in whole steps of four sub-blocks (one weight-scale block each for the scaled kinds)
        const int per = (((KT_all + p.ksplit - 1) / p.ksplit) + 3) & ~3;
        kt0 = (int)blockIdx.z * per;
        KT = max(0, min(per, KT_all - kt0));
    }
    const int nsteps = (KT + 3) >> 2;
    const int n0 = blockIdx.x * MD_BN, m_start = blockIdx.y * BM, m_end = min(p.M, m_start + BM);

    // LDS map
    uint8_t* const a_st = lds;                              // [MD_NA][MD_A]
    uint8_t* const b_st = lds + MD_NA * MD_A;               // [MD_NBS][MD_B]
    uint8_t* const s_st = lds + MD_NA * MD_A + MD_NBS * MD_B;        // [MD_NA][MD_S]
    float* const bsl = (float*)(lds + md_stages(MT));       // weight scale of the tile's column block per sub-block
    uint8_t* const w4tab = lds + md_stages(MT) + D_MAX_KT * 4;   // [s4 | z4][sub-block][64 rows] bytes

    // ---- per-thread source offsets.  A piece = 8 rows x 128 bytes = what one load instruction of a wave covers
    // (lane: row lane >> 3, 16-byte chunk lane & 7, XOR-swizzled with (row >> 1) & 7 on the global side so that
    // the fragment reads are conflict-free).  Wave w moves pieces MT w .. MT w + MT - 1 of the 4 x 2 MT activation
    // pieces of a step: piece = (sub-block, row group).
    const int row8 = lane >> 3;
    uint32_t aoff[MT], alds[MT];
    int asub[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int pq = MT * wave + i, sub = pq / (2 * MT), row = 8 * (pq % (2 * MT)) + row8;
        const uint32_t chunk = (uint32_t)((lane & 7) ^ ((row >> 1) & 7)) * 16u;
        aoff[i] = (uint32_t)min(m_start + row, m_end - 1) * (uint32_t)K + chunk;
        alds[i] = (uint32_t)(sub * (BM * 128) + 8 * (pq % (2 * MT)) * 128);     // + lane * 16 by the hardware
        asub[i] = sub;
    }
    // weights: one wave per packed row (eight weight rows): lane l takes words 4 l .. 4 l + 3 of sub-blocks l >> 5
    // (load 0) and 2 + (l >> 5) (load 1) of the step's 512 words
    const uint32_t boff = (uint32_t)min((n0 >> 3) + wave, (N >> 3) - 1) * (uint32_t)(p.K * 4) + (uint32_t)(lane & 31) * 16u;
    constexpr uint32_t SSZ = AS16 ? 2u : 4u;                // bytes per activation scale
    const uint32_t soff = (uint32_t)min(m_start + min(lane, BM - 1), m_end - 1) * (uint32_t)KT_all * SSZ;

    // sub-block `sub` of step s, clamped to the last one of the range: requests past the end repeat the last step
    auto phys = [&](int s) { return min(s, nsteps - 1); };
    auto kblock = [&](int s, int sub) { return kt0 + min(4 * phys(s) + sub, KT - 1); };

    auto issue_a = [&](int s) {
        const uint32_t st = lds_base + (uint32_t)(s % MD_NA) * MD_A;
#pragma unroll
        for (int i = 0; i < MT; ++i) dma16(st + alds[i], aoff[i], p.a + (int64_t)kblock(s, asub[i]) * 128);
        const uint32_t ss = lds_base + MD_NA * MD_A + MD_NBS * MD_B + (uint32_t)(s % MD_NA) * MD_S + (uint32_t)(wave & 3) * 256u;
        if constexpr (AS16) dma2(ss, soff, (const uint8_t*)p.a_s + (int64_t)kblock(s, wave & 3) * 2);
        else dma4(ss, soff, (const uint8_t*)p.a_s + (int64_t)kblock(s, wave & 3) * 4);
    };
    // ring of weight registers: slot = step % 4
    v4i ring[MD_RING][NB];
    auto issue_b = [&](v4i (&rs)[NB], int s) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            // lane-dependent sub-block: the two halves of the wave read different 128-word runs of the row
            const int kb0 = kblock(s, 2 * i), kb1 = kblock(s, 2 * i + 1);
            const uint32_t off = boff + (uint32_t)((lane >> 5) ? kb1 - kb0 : 0) * 512u;
            rs[i] = asm_load_b128(off, (const uint8_t*)p.b + (int64_t)kb0 * 512);
        }
    };
    // the loads of slot `slot` have landed when at most `younger` loads issued after them are in flight
    auto ring_ready = [&](v4i (&rs)[NB], auto younger_c) __attribute__((always_inline)) {
        constexpr int Y = decltype(younger_c)::value;
        asm volatile("s_waitcnt vmcnt(%2)" : "+v"(rs[0]), "+v"(rs[1]) : "n"(Y) : "memory");
    };
    // ring slot -> weight stage s & 1 (nobody has read that stage since the barrier of step s - 1), as int8 rows
    // (q - z4) * s4.  Lane: words 4 kc .. 4 kc + 3 (kc = lane & 31) of sub-block 2 i + (lane >> 5); packed row = wave;
    // row j of the packed row is tile column 8 wave + j.
    auto produce = [&](const v4i (&rs)[NB], int s) __attribute__((always_inline)) {
        uint8_t* st = b_st + (s % MD_NBS) * MD_B;
        const int kc = lane & 31;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int sub = 2 * i + (lane >> 5);
            const int kb = min(4 * phys(s) + sub, KT - 1);
            const uint8_t* tabk = w4tab + kb * 64 + 8 * wave;
            unsigned sp[4], cp[4], rows[8];
            w4a8_row_consts(*(const uint2*)tabk, *(const uint2*)(tabk + 64 * KT), sp, cp);
            w4a8_words_to_i8(rs[i], sp, cp, rows);
            uint8_t* dst = st + sub * (MD_BN * 128) + (kc & 3) * 4;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int R = 8 * wave + j;
                *(unsigned*)(dst + R * 128 + (((kc >> 2) ^ ((R >> 1) & 7)) * 16)) = rows[j];
            }
        }
    };

    // acc[i][j][q] = C[row 16 i + r][column 32 wn + 16 j + 4 g + q] summed over this wave's sub-blocks
    v4f acc[MT][2];
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[i][0] = acc[i][1] = (v4f){0.f, 0.f, 0.f, 0.f};

    // fragment read offsets inside a 16-row slab: chunks g and g + 4 of row r, swizzled
    const int lo = r * 128 + ((g ^ ((r >> 1) & 7)) * 16);
    const int hi = r * 128 + (((g + 4) ^ ((r >> 1) & 7)) * 16);
    auto ldfrag = [&](const uint8_t* base) {
        const v4i x = *(const v4i*)(base + lo), y = *(const v4i*)(base + hi);
        return (v8i){x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]};
    };
    auto compute = [&](int s) {
        const uint8_t* As = a_st + (s % MD_NA) * MD_A + kq * (BM * 128);
        const uint8_t* Bs = b_st + (s % MD_NBS) * MD_B + kq * (MD_BN * 128) + (wn * 32) * 128;
        const int kb = 4 * phys(s) + kq;
        const bool live = kb < KT;                         // wave-uniform: sub-blocks past the range add nothing
        // activation fragments one tile row ahead of their use
        v8i bf[2], af[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) bf[j] = ldfrag(Bs + j * 2048);
        af[0] = ldfrag(As);
        const float* Ss = (const float*)(s_st + (s % MD_NA) * MD_S) + kq * 64 + r;
        const float bs = live ? bsl[min(kb, KT - 1)] : 0.f;
        float sa[MT];
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            if constexpr (AS16) {
                const unsigned raw = ((const unsigned*)Ss)[16 * i];
                sa[i] = (p.s_dtype == LLMK_F16 ? f16_to_f32((unsigned short)raw) : bf16_to_f32((unsigned short)raw)) * bs;
            } else {
                sa[i] = Ss[16 * i] * bs;
            }
        }
        // the products of tile row i are scaled and accumulated while the matrix instructions of row i + 1 run
        v4f t[2][2];
#pragma unroll
        for (int i = 0; i <= MT; ++i) {
            if (i + 1 < MT) af[(i + 1) & 1] = ldfrag(As + (i + 1) * 2048);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (i < MT) t[i & 1][j] = step_dot<KIND>(bf[j], af[i & 1]);
                if (i > 0) acc[i - 1][j] += t[(i - 1) & 1][j] * sa[i - 1];
            }
            // nothing moves across a tile row: the lag of one row between product and accumulation stays, and
            // the fragments of at most two rows are live
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    const std::integral_constant<int, 0> c0;
    const std::integral_constant<int, (MD_RING - 2) * NB> cpro;
    const std::integral_constant<int, NB> cnb;

    // ---- prologue: activations of step 0, weights of steps 0, 1, 2; tables by ordinary loads meanwhile
    issue_a(0);
    md_static_for<0, MD_RING - 1>([&](auto ic) __attribute__((always_inline)) { issue_b(ring[ic.value], ic.value); });
    const int64_t bs_row = (int64_t)(n0 >> 7) * KT_all + kt0;
    for (int i = tid; i < KT; i += MD_THREADS) bsl[i] = ld_scale(p.b_s, bs_row + i, p.s_dtype);
    for (int i = tid; i < 64 * KT; i += MD_THREADS) {
        const int row = i / KT, kk = i - row * KT;
        const int64_t at = (int64_t)min(n0 + row, N - 1) * KT_all + kt0 + kk;
        w4tab[kk * 64 + row] = (uint8_t)p.w4_s4[at];
        w4tab[(KT + kk) * 64 + row] = (uint8_t)p.w4_z4[at];
    }
    __syncthreads();                                        // the table is read by produce()
    ring_ready(ring[0], cpro);
    produce(ring[0], 0);

    // One step: wait for the activations of step s (requested a step ago; only the NB weight loads issued after
    // them may stay in flight; with four ring slots that also vouches for slot s + 1, requested two steps ago),
    // meet the others, request the activations of step s + 1 and the weights of step s + MD_RING - 1, multiply
    // step s, and move the weights of step s + 1 from the ring into the other weight stage.
    auto step = [&](auto slot_c, int s) __attribute__((always_inline)) {
        constexpr int slot = decltype(slot_c)::value;
        // (scheduling fences: without them the compiler carries the matrix instructions of a step across the next
        // barrier, with all fragments of two steps live, and spills)
        __builtin_amdgcn_sched_barrier(0);
        ring_ready(ring[(slot + 1) % MD_RING], cnb);
        __builtin_amdgcn_s_waitcnt(0xc07f);                 // lgkmcnt(0): this wave's LDS writes of produce() are done
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        issue_a(s + 1);
        issue_b(ring[(slot + MD_RING - 1) % MD_RING], s + MD_RING - 1);
        __builtin_amdgcn_sched_barrier(0);
        compute(s);
        __builtin_amdgcn_sched_barrier(0);
        produce(ring[(slot + 1) % MD_RING], s + 1);
        __builtin_amdgcn_sched_barrier(0);
    };
    int s = 0;
    for (int rd = nsteps / MD_RING; rd > 0; --rd) {
        md_static_for<0, MD_RING>([&](auto ic) __attribute__((always_inline)) { step(ic, s + ic.value); });
        s += MD_RING;
    }
    md_static_nested<0, MD_RING - 1>(nsteps % MD_RING, [&](auto ic) __attribute__((always_inline)) { step(ic, s + ic.value); });
    // everything requested has landed (also the repeated loads past the end) before the stages are reused
    md_static_for<0, MD_RING>([&](auto ic) __attribute__((always_inline)) { ring_ready(ring[ic.value], c0); });
    __syncthreads();

    // ---- the four sub-block sums of every output meet in LDS: red[kq][row][column], rows of 68 floats
    float* red = (float*)lds;
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
            *(v4f*)(red + (kq * BM + 16 * i + r) * MD_RED_ROW + wn * 32 + 16 * j + 4 * g) = acc[i][j];
    __syncthreads();
    // thread: row tid >> 3, columns 8 (tid & 7) .. + 7
    const int orow = tid >> 3, ocol = 8 * (tid & 7);
    if (orow >= BM) return;
    const int m = m_start + orow, n = n0 + ocol;
    if (m >= m_end || n >= N) return;
    v4f sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float* src = red + (q * BM + orow) * MD_RED_ROW + ocol;
        sa += *(const v4f*)src;
        sb += *(const v4f*)(src + 4);
    }
    const bool split = p.ksplit > 1;
    void* cout = split ? (void*)(p.partial + (int64_t)blockIdx.z * p.M * N) : p.c;
    const int cdt = split ? LLMK_F32 : p.c_dtype;
    const int esz = cdt == LLMK_F32 ? 4 : 2;
    const bool vec_ok = ((((uintptr_t)cout) & 15) == 0) && (((int64_t)N * esz) % 16 == 0);
    const int nv = N - n;
    const int64_t off = (int64_t)m * N + n;
    if (cdt == LLMK_BF16) store_run8<LLMK_BF16>(cout, off, sa, sb, nv, vec_ok);
    else if (cdt == LLMK_F16) store_run8<LLMK_F16>(cout, off, sa, sb, nv, vec_ok);
    else store_run8<LLMK_F32>(cout, off, sa, sb, nv, vec_ok);
}

// ------------------------------------------------------------------------------------------------------------
// Producer / consumer form of the same tile for 8- and 16-bit operands.  A cycle count of the kernel above (per wave and
// phase) showed that it never waits for data: what a step costs is ISSUING its loads.  The CU's vector-memory path takes
// about 16 cycles per 1 KB instruction (64 bytes per clock, the 110 GB/s per CU), a step of a 64 x 64 tile is 64 such
// instructions (about 1100 cycles), and a wave that is issuing loads cannot multiply: with all eight waves issuing behind
// the barrier, then multiplying, then writing weight rows, the phases add up to 2900 cycles per step.  Here the roles are
// split so that they overlap:
//   waves 4 .. 7 (producers, one per SIMD): wave 4 + q moves sub-block q of the step for BOTH operands: activation rows
//       by direct-to-LDS loads one step ahead, weight rows by hand-issued register loads MDP_RB steps ahead (ring of
//       MDP_RB register sets), written into the weight stage one step ahead.  They issue loads all the time.
//   waves 0 .. 3 (consumers, one per SIMD): wave q multiplies sub-block q of the step for the whole 16 MT x 64 tile
//       (4 MT matrix instructions for MT + 4 fragment reads) and never touches global memory inside the loop.
// Two stages (activations | weights | activation-scale column); one barrier per step, after which the stage just filled
// is complete and the one just multiplied is free.  The four sub-block sums meet in LDS at the end as before.
// WIDE: the same roles on a 16 MT x 128 tile with K steps of 256 bytes = two sub-blocks (MT = 4 or 8), for weights with
// more 64-column tiles than CUs: producer 4 + q moves sub-block q & 1 of the step for the row half and the column half
// q >> 1, consumer q multiplies sub-block q & 1 for the column half q >> 1; two partial sums per output meet at the end.
constexpr int MDP_RB = 3;
constexpr int mdp_bn(bool wide) { return wide ? 128 : 64; }
constexpr int mdp_nsub(bool wide) { return wide ? 2 : 4; }                       // 128-byte sub-blocks per K step
constexpr int mdp_a(int mt, bool wide) { return mdp_nsub(wide) * 16 * mt * 128; }
constexpr int mdp_stage(int mt, bool wide = false) { return mdp_a(mt, wide) + MD_B + MD_S; }
constexpr int mdp_red(int mt, bool wide) { return mdp_nsub(wide) * 16 * mt * (mdp_bn(wide) + 4) * 4; }
constexpr int mdp_lds(int mt, bool wide = false) {
    return (2 * mdp_stage(mt, wide) > mdp_red(mt, wide) ? 2 * mdp_stage(mt, wide) : mdp_red(mt, wide)) + D_MAX_KT * 4;
}

template <int KIND, int MT, bool AS16 = false, bool WIDE = false>
__global__ __launch_bounds__(MD_THREADS) void gemm_mid_pc_kernel(DirectArgs p) {
    static_assert(WIDE ? (MT == 8 || MT == 4) : (MT == 4 || MT == 2), "tile rows");
    constexpr int BN = mdp_bn(WIDE), NSUB = mdp_nsub(WIDE), RED_ROW = BN + 4;
    static_assert(BN * NSUB * 128 == MD_B && RED_ROW == (WIDE ? 132 : MD_RED_ROW), "weight stage of 32 KB");
    static_assert(KIND == K_FP8_BLOCK || KIND == K_I8_BLOCK || KIND == K_I8_ROWCOL || KIND == K_F16 || KIND == K_BF16 || KIND == K_W4NK,
                  "8- and 16-bit operands, or fp16 activations with row-packed 4-bit weights");
    constexpr int BM = 16 * MT;
    // K_W4NK: the producers load packed words [N, K/8] and their group scales (fp16, groups of 64 * 2^j elements) and write
    // fp16 weight rows (q - 8) * scale into the weight stage; the rest is the fp16 kind
    constexpr bool W4NK = (KIND == K_W4NK);
    constexpr bool SCALED = (KIND == K_FP8_BLOCK || KIND == K_I8_BLOCK);
    constexpr bool ROWCOL = (KIND == K_I8_ROWCOL);
    constexpr int ESZ = (KIND == K_F16 || KIND == K_BF16 || W4NK) ? 2 : 1;
    constexpr int MD_A = mdp_a(MT, WIDE), STAGE = mdp_stage(MT, WIDE);
    constexpr int RB = MDP_RB;
    constexpr int NPA = 2 * MT * NSUB / 4;                  // activation pieces per producer wave and step
    constexpr int NAP = NPA + (SCALED ? 1 : 0);             // direct-to-LDS loads per producer wave and step
    constexpr int NBR = W4NK ? 2 : 8;                       // 16-byte weight registers per producer lane and step
    constexpr int NBP = W4NK ? 4 : 8;                       // register loads per producer wave and step (K_W4NK: + two scales)
    constexpr int LP = NAP + NBP;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4, q = wave & 3;
    const bool producer = wave >= 4;
    const int ksub = WIDE ? (q & 1) : q, half = WIDE ? (q >> 1) : 0;     // sub-block of the step, row / column half
    const int N = p.N;
    const int K = p.K * ESZ;                                // row length in bytes
    const int KT_all = K >> 7;                              // 128-byte sub-blocks per row
    int kt0 = 0, KT = KT_all;                               // sub-blocks [kt0, kt0 + KT) of this workgroup
    if (p.ksplit > 1) {
        const int per = (((KT_all + p.ksplit - 1) / p.ksplit) + 3) & ~3;
        kt0 = (int)blockIdx.z * per;
        KT = max(0, min(per, KT_all - kt0));
    }
    const int nsteps = (KT + NSUB - 1) / NSUB;
    const int n0 = blockIdx.x * BN, m_start = blockIdx.y * BM, m_end = min(p.M, m_start + BM);
    float* const bsl = (float*)(lds + (mdp_lds(MT, WIDE) - D_MAX_KT * 4));

    // acc[i][j][e] = C[row 16 i + r][column 64 half + 16 j + 4 g + e] summed over sub-block ksub of all steps (consumers)
    v4f acc[MT][4];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

    if (producer) {
        // ---- source offsets.  A piece = 8 rows x 128 bytes = one load instruction of the wave (lane: row lane >> 3,
        // 16-byte chunk lane & 7); the chunk index is XOR-swizzled with (row >> 1) & 7, on the global side for the
        // direct-to-LDS loads and on the LDS side for the weight rows, so that the fragment reads are conflict-free.
        const int row8 = lane >> 3;
        uint32_t aoff[NPA], boff[NBR], blds[NBR], w4_soff[2] = {0, 0}, w4_chunk[2] = {0, 0};
        int w4_shift = 0;
        constexpr int SEGS = 4 * NSUB / 2;                  // K_W4NK: 32-weight segments of a row per step (8 or 4)
        const int w4_sub = (tid & (SEGS - 1)) >> 1;         // K_W4NK: sub-block of this lane's 32 weights
        const int arow0 = half * (8 * NPA);                 // WIDE: the two producers of a sub-block halve the rows
#pragma unroll
        for (int i = 0; i < NPA; ++i) {
            const int row = arow0 + 8 * i + row8;
            aoff[i] = (uint32_t)min(m_start + row, m_end - 1) * (uint32_t)K + (uint32_t)((lane & 7) ^ ((row >> 1) & 7)) * 16u;
        }
#pragma unroll
        for (int i = 0; i < NBR; ++i) {
            if constexpr (W4NK) {
                // producer thread t = 0 .. 255: the 32 weights k = 32 seg .. + 31 (seg = t & 7) of the step's 256 of rows
                // t >> 3 and 32 + (t >> 3): 16 bytes of packed words each, four 16-byte chunks of the fp16 row of
                // sub-block seg >> 1, and the group scale of those weights
                // (WIDE: 128 weights per row and step, four segments; rows t >> 2 and 64 + (t >> 2))
                const int row = ((tid - 256) / SEGS) + (256 / SEGS) * i, seg = tid & (SEGS - 1);
                const uint32_t n = (uint32_t)min(n0 + row, N - 1);
                boff[i] = n * (uint32_t)(p.K >> 1) + (uint32_t)(seg & 1) * 16u;       // + 32 bytes per sub-block
                w4_soff[i] = n * (uint32_t)(p.K / p.group) * 2u;
                blds[i] = (uint32_t)(MD_A + (seg >> 1) * (BN * 128) + row * 128);
                w4_chunk[i] = (uint32_t)(((4 * (seg & 1)) ^ ((row >> 1) & 7)) * 16);  // first chunk; chunk c is at ^ (c * 16)
            } else {
                const int row = 64 * half + 8 * i + row8;
                boff[i] = (uint32_t)min(n0 + row, N - 1) * (uint32_t)K + (uint32_t)(lane & 7) * 16u;
                blds[i] = (uint32_t)(MD_A + ksub * (BN * 128) + row * 128 + (((lane & 7) ^ ((row >> 1) & 7)) * 16));
            }
        }
        if constexpr (W4NK) w4_shift = __builtin_ctz((unsigned)(p.group >> 6));
        auto kblock_sub = [&](int s, int sub) { return kt0 + min(NSUB * min(max(s, 0), nsteps - 1) + sub, KT - 1); };
        constexpr uint32_t SSZ = AS16 ? 2u : 4u;
        // scale column of a sub-block: 64 rows per producer (WIDE: the two producers of the sub-block take 64 rows each)
        const uint32_t soff = (uint32_t)min(m_start + min(lane + 64 * half, BM - 1), m_end - 1) * (uint32_t)KT_all * SSZ;
        // sub-block ksub of step s, clamped to the last one of the range (requests past the end repeat it)
        auto kblock = [&](int s) { return kt0 + min(NSUB * min(max(s, 0), nsteps - 1) + ksub, KT - 1); };
        auto issue_a = [&](int s) {
            const uint32_t st = lds_base + (uint32_t)(s & 1) * STAGE;
            const int kb = kblock(s);
#pragma unroll
            for (int i = 0; i < NPA; ++i) dma16(st + (uint32_t)(ksub * (BM * 128) + (arow0 + 8 * i) * 128), aoff[i], p.a + (int64_t)kb * 128);
            if constexpr (SCALED) {
                const uint32_t ss = st + MD_A + MD_B + (uint32_t)(WIDE ? 2 * ksub + half : q) * 256u;
                if constexpr (AS16) dma2(ss, soff, (const uint8_t*)p.a_s + (int64_t)kb * 2);
                else dma4(ss, soff, (const uint8_t*)p.a_s + (int64_t)kb * 4);
            }
        };
        v4i ring[RB][NBR];
        unsigned ringsc[RB][2] = {};                        // K_W4NK: group scales of the slot's weights (fp16 bits)
        auto issue_b = [&](v4i (&rs)[NBR], unsigned (&rsc)[2], int s) __attribute__((always_inline)) {
            if constexpr (W4NK) {
                // lane-dependent sub-block (the eight lanes of a row cover the four sub-blocks of the step)
                const int kb0 = kblock_sub(s, 0), kb = kblock_sub(s, w4_sub);
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    rs[i] = asm_load_b128(boff[i] + (uint32_t)(kb - kb0) * 32u, (const uint8_t*)p.b + (int64_t)kb0 * 32);
                    rsc[i] = asm_load_u16(w4_soff[i] + (uint32_t)(kb >> w4_shift) * 2u, p.b_s);
                }
            } else {
                const uint8_t* base = p.b + (int64_t)kblock(s) * 128;
#pragma unroll
                for (int i = 0; i < NBR; ++i) rs[i] = asm_load_b128(boff[i], base);
            }
        };
        auto ring_ready = [&](v4i (&rs)[NBR], unsigned (&rsc)[2], auto younger_c) __attribute__((always_inline)) {
            constexpr int Y = decltype(younger_c)::value;
            if constexpr (W4NK)
                asm volatile("s_waitcnt vmcnt(%4)" : "+v"(rs[0]), "+v"(rs[1]), "+v"(rsc[0]), "+v"(rsc[1]) : "n"(Y) : "memory");
            else
                asm volatile("s_waitcnt vmcnt(%8)" : "+v"(rs[0]), "+v"(rs[1]), "+v"(rs[2]), "+v"(rs[3]), "+v"(rs[4]), "+v"(rs[5]), "+v"(rs[6]), "+v"(rs[7]) : "n"(Y) : "memory");
        };
        auto write_b = [&](const v4i (&rs)[NBR], const unsigned (&rsc)[2], int s) __attribute__((always_inline)) {
            uint8_t* st = lds + (s & 1) * STAGE;
            if constexpr (W4NK) {
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const v2h sc = w4_as_h2(rsc[i] | (rsc[i] << 16));
#pragma unroll
                    for (int c = 0; c < 4; ++c) *(v4i*)(st + blds[i] + (w4_chunk[i] ^ (uint32_t)(c * 16))) = w4_word_to_f16x8((unsigned)rs[i][c], sc);
                }
            } else {
#pragma unroll
                for (int i = 0; i < NBR; ++i) *(v4i*)(st + blds[i]) = rs[i];
            }
        };
        static_assert(RB == 3, "the prologue below spells out three ring slots");
        const std::integral_constant<int, 0> c0;
        const std::integral_constant<int, (RB - 1) * LP> cb;
        const std::integral_constant<int, (RB - 1) * NBP> cb_pro;      // step -1: only weight requests behind those of step 0
        const std::integral_constant<int, LP + NBP> cb_first;          // step 0: one full step and the weights of step 2
        // Step s of a producer, behind barrier s: request the activations of step s + 1 and the weights of step s + RB; the
        // weights of step s + 1, requested RB - 1 steps ago, have landed when only the loads of the steps since are in
        // flight: write them into the other stage; the activations just requested have landed when only the NBP weight
        // loads behind them are in flight; barrier s + 1.
        auto pstep = [&](auto slot_c, auto count_c, int s) __attribute__((always_inline)) {
            constexpr int slot = decltype(slot_c)::value;    // = s mod RB
            __builtin_amdgcn_sched_barrier(0);
            issue_a(s + 1);
            issue_b(ring[slot], ringsc[slot], s + RB);
            __builtin_amdgcn_sched_barrier(0);
            ring_ready(ring[(slot + 1) % RB], ringsc[(slot + 1) % RB], count_c);
            write_b(ring[(slot + 1) % RB], ringsc[(slot + 1) % RB], s + 1);
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("s_waitcnt vmcnt(%0)" : : "n"(NBP) : "memory");
            __builtin_amdgcn_s_waitcnt(0xc07f);             // lgkmcnt(0): the weight rows are in LDS
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
        };
        // prologue: activations of step 0, weights of steps 0 .. RB - 1; the weights of step 0 have landed when only the
        // two weight requests behind them are in flight (the activations, requested before them, then have too)
        issue_a(0);
        md_static_for<0, RB>([&](auto ic) __attribute__((always_inline)) { issue_b(ring[ic.value], ringsc[ic.value], ic.value); });
        ring_ready(ring[0], ringsc[0], cb_pro);
        write_b(ring[0], ringsc[0], 0);
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __syncthreads();                                    // barrier 0
        __builtin_amdgcn_sched_barrier(0);
        // step 0 has a wait count of its own (no activation requests in the prologue steps before it), then rounds of the
        // three ring slots starting at slot 1
        int s = 0;
        if (nsteps > 0) {
            pstep(std::integral_constant<int, 0>{}, cb_first, 0);
            s = 1;
            for (int rd = (nsteps - 1) / RB; rd > 0; --rd) {
                md_static_for<0, RB>([&](auto ic) __attribute__((always_inline)) { pstep(std::integral_constant<int, (1 + ic.value) % RB>{}, cb, s + ic.value); });
                s += RB;
            }
            md_static_nested<0, RB - 1>((nsteps - 1) % RB, [&](auto ic) __attribute__((always_inline)) { pstep(std::integral_constant<int, (1 + ic.value) % RB>{}, cb, s + ic.value); });
        }
        // everything requested has landed (also the repeated loads past the end) before the stages are reused
        md_static_for<0, RB>([&](auto ic) __attribute__((always_inline)) { ring_ready(ring[ic.value], ringsc[ic.value], c0); });
    } else {
        // ---- consumer: fragment read offsets inside a 16-row slab: chunks g and g + 4 of row r, swizzled
        const int lo = r * 128 + ((g ^ ((r >> 1) & 7)) * 16);
        const int hi = r * 128 + (((g + 4) ^ ((r >> 1) & 7)) * 16);
        auto ldfrag = [&](const uint8_t* base) {
            const v4i x = *(const v4i*)(base + lo), y = *(const v4i*)(base + hi);
            return (v8i){x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]};
        };
        // weight scales of the tile's column block, while the producers request the first steps; barrier 0 publishes them
        if constexpr (SCALED) {
            const int64_t bs_row = (int64_t)(n0 >> 7) * KT_all + kt0;
            for (int i = tid; i < KT; i += MD_THREADS / 2) bsl[i] = ld_scale(p.b_s, bs_row + i, p.s_dtype);
        }
        __syncthreads();                                    // barrier 0
        for (int s = 0; s < nsteps; ++s) {
            const uint8_t* st = lds + (s & 1) * STAGE;
            const uint8_t* As = st + ksub * (BM * 128);
            const uint8_t* Bs = st + MD_A + ksub * (BN * 128) + half * (64 * 128);
            const int kb = NSUB * s + ksub;
            const bool live = kb < KT;                     // wave-uniform: sub-blocks past the range add nothing
            v8i bf[4], af[2];
#pragma unroll
            for (int j = 0; j < 4; ++j) bf[j] = ldfrag(Bs + j * 2048);
            af[0] = ldfrag(As);
            if constexpr (SCALED) {
                const float* Ss = (const float*)(st + MD_A + MD_B) + ksub * (WIDE ? 128 : 64) + r;
                const float bs = live ? bsl[min(kb, KT - 1)] : 0.f;
                float sa[MT];
#pragma unroll
                for (int i = 0; i < MT; ++i) {
                    if constexpr (AS16) {
                        const unsigned raw = ((const unsigned*)Ss)[16 * i];
                        sa[i] = (p.s_dtype == LLMK_F16 ? f16_to_f32((unsigned short)raw) : bf16_to_f32((unsigned short)raw)) * bs;
                    } else {
                        sa[i] = Ss[16 * i] * bs;
                    }
                }
                // the products of tile row i are scaled and accumulated while the matrix instructions of row i + 1 run
                v4f t[2][4];
#pragma unroll
                for (int i = 0; i <= MT; ++i) {
                    if (i + 1 < MT) af[(i + 1) & 1] = ldfrag(As + (i + 1) * 2048);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (i < MT) t[i & 1][j] = step_dot<KIND>(bf[j], af[i & 1]);
                        if (i > 0) acc[i - 1][j] += t[(i - 1) & 1][j] * sa[i - 1];
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                const v8i zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (int i = 0; i < MT; ++i) {
                    if (i + 1 < MT) af[(i + 1) & 1] = ldfrag(As + (i + 1) * 2048);
                    const v8i a = live ? af[i & 1] : zero8;
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[i][j] = mma_plain<KIND>(bf[j], a, acc[i][j]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();                                // barrier s + 1: this stage is free, the other one complete
        }
    }
    __syncthreads();

    // ---- the NSUB sub-block sums of every output meet in LDS: red[sub-block][row][column], rows of BN + 4 floats
    float* red = (float*)lds;
    if (!producer) {
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *(v4f*)(red + (ksub * BM + 16 * i + r) * RED_ROW + 64 * half + 16 * j + 4 * g) = acc[i][j];
    }
    __syncthreads();
    // thread: columns 8 (tid % (BN / 8)) .. + 7 of row tid / (BN / 8), then the rows 4096 / BN further on
    constexpr int RUNS = BN / 8, ROWS_PASS = MD_THREADS / RUNS;
    const bool split = p.ksplit > 1;
    void* cout = split ? (void*)(p.partial + (int64_t)blockIdx.z * p.M * N) : p.c;
    const int cdt = split ? LLMK_F32 : p.c_dtype;
    const int esz = cdt == LLMK_F32 ? 4 : 2;
    const bool vec_ok = ((((uintptr_t)cout) & 15) == 0) && (((int64_t)N * esz) % 16 == 0);
    const int ocol = 8 * (tid % RUNS), n = n0 + ocol, nv = N - n;
    if (n >= N) return;
#pragma unroll
    for (int pass = 0; pass < (BM + ROWS_PASS - 1) / ROWS_PASS; ++pass) {
        const int orow = pass * ROWS_PASS + tid / RUNS;
        const int m = m_start + orow;
        if (orow >= BM || m >= m_end) continue;
        v4f sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
        if constexpr (ROWCOL) {
            v4i ia = {0, 0, 0, 0}, ib = {0, 0, 0, 0};
#pragma unroll
            for (int k = 0; k < NSUB; ++k) {
                const float* src = red + (k * BM + orow) * RED_ROW + ocol;
                ia += *(const v4i*)src;
                ib += *(const v4i*)(src + 4);
            }
            __builtin_memcpy(&sa, &ia, 16);
            __builtin_memcpy(&sb, &ib, 16);
        } else {
#pragma unroll
            for (int k = 0; k < NSUB; ++k) {
                const float* src = red + (k * BM + orow) * RED_ROW + ocol;
                sa += *(const v4f*)src;
                sb += *(const v4f*)(src + 4);
            }
        }
        const int64_t off = (int64_t)m * N + n;
        if constexpr (ROWCOL) {
            // (a K slice leaves its int32 sums, bit for bit, in the fp32 partial buffer: the summing pass adds them as
            // integers and scales once, so the result does not depend on the split)
            if (!split) {
                rowcol_epilogue8(p, sa, sb, m, off, n, nv);
                if (!p.c) continue;
            }
        }
        if (cdt == LLMK_BF16) store_run8<LLMK_BF16>(cout, off, sa, sb, nv, vec_ok);
        else if (cdt == LLMK_F16) store_run8<LLMK_F16>(cout, off, sa, sb, nv, vec_ok);
        else store_run8<LLMK_F32>(cout, off, sa, sb, nv, vec_ok);
    }
}

// K slices of the mid-size kernel: as many as bring the grid to about one workgroup per CU, in whole steps of 512
// bytes, each slice at least four steps long; 1 = no split.
inline int mid_splitk(int64_t tiles, int64_t kbytes) {
    if (tiles >= 3 * LLMK_CUS / 4) return 1;
    int64_t z = LLMK_CUS / tiles;
    const int64_t steps = kbytes >> 9;
    if (z > steps / 4) z = steps / 4;
    return (int)(z > 8 ? 8 : (z < 1 ? 1 : z));
}

// Shape of a mid-size launch: tile height (16 mt rows) and K slices.  The 32-row tile when the 64-row tile would leave
// more than half of the CUs without a workgroup.
struct MidPlan {
    int mt, z;
    int64_t tiles;
};
inline MidPlan mid_plan(int64_t M, int64_t N, int64_t kbytes) {
    MidPlan pl;
    const int64_t gx = (N + MD_BN - 1) / MD_BN;
    const int64_t t4 = ((M + 63) / 64) * gx, t2 = ((M + 31) / 32) * gx;
    pl.mt = (t4 <= LLMK_CUS / 2 && t2 > t4) ? 2 : 4;
    pl.tiles = pl.mt == 4 ? t4 : t2;
    pl.z = mid_splitk(pl.tiles, kbytes);
    return pl;
}

// The 128-column form: 64-row tiles while they fit one round of workgroups, else 128-row tiles; K slices as above.
inline MidPlan midw_plan(int64_t M, int64_t N, int64_t kbytes) {
    MidPlan pl;
    const int64_t gx = (N + 127) / 128;
    const int64_t t4 = ((M + 63) / 64) * gx, t8 = ((M + 127) / 128) * gx;
    pl.mt = t4 <= LLMK_CUS ? 4 : 8;
    pl.tiles = pl.mt == 4 ? t4 : t8;
    pl.z = mid_splitk(pl.tiles, kbytes);
    return pl;
}

// Eligibility: 32-bit source offsets, whole 128-byte sub-blocks, scale table size (as dma_eligible), and for the
// K_W4A8 kind room for its table behind the stages.
template <int KIND>
inline bool mid_eligible(const DirectArgs& p, int mt, int ksplit) {
    constexpr int ESZ = (KIND == K_F16 || KIND == K_BF16 || KIND == K_W4NK) ? 2 : 1;
    if (!dma_eligible(p, ESZ)) return false;
    if (KIND == K_W4NK && (p.group < 64 || (p.group & (p.group - 1)))) return false;      // groups of 64 * 2^j elements
    const int KT_all = (p.K * ESZ) >> 7;
    const int per = ksplit > 1 ? ((((KT_all + ksplit - 1) / ksplit) + 3) & ~3) : KT_all;
    return md_lds(mt, KIND == K_W4A8 ? per : 0) <= D_LDS_MAX;
}

// p.a_s: fp32, or with AS16 the 16-bit scales of dtype p.s_dtype as the caller passed them; p.s_dtype describes b_s
// (and those).  p.ksplit / p.partial select the K split.
template <int KIND, int MT, bool AS16 = false, bool WIDE = false>
int launch_mid(const DirectArgs& p, hipStream_t stream, const char* name) {
    static std::atomic<uint64_t> configured{0};
    constexpr bool W4 = (KIND == K_W4A8);
    static_assert(!(W4 && WIDE), "the 128-column form exists for the producer / consumer kernel only");
    // the producer / consumer form, except for w4a8 (whose expansion is vector-ALU work that wants all eight waves)
    auto kern = [] {
        if constexpr (W4) return gemm_mid_kernel<KIND, MT, AS16>;
        else return gemm_mid_pc_kernel<KIND, MT, AS16, WIDE>;
    }();
    constexpr int ESZ = (KIND == K_F16 || KIND == K_BF16 || KIND == K_W4NK) ? 2 : 1;
    const int KT_all = (p.K * ESZ) >> 7;
    const bool split = p.ksplit > 1 && p.partial;
    const int per = split ? ((((KT_all + p.ksplit - 1) / p.ksplit) + 3) & ~3) : KT_all;
    const int lds_bytes = W4 ? md_lds(MT, per) : mdp_lds(MT, WIDE);
    if (lds_bytes > D_LDS_MAX) LLMK_FAIL(LLMK_ERR_SHAPE, "%s: %d bytes of LDS needed", name, lds_bytes);
    if (int rc = llmk_reserve_lds((const void*)kern, D_LDS_MAX, configured, name)) return rc;
    // slices that would start past the end of K are not launched
    const int z = split ? (KT_all + per - 1) / per : 1;
    DirectArgs q = p;
    q.ksplit = split ? p.ksplit : 1;
    constexpr int BN = mdp_bn(WIDE);
    dim3 grid((unsigned)((p.N + BN - 1) / BN), (unsigned)((p.M + 16 * MT - 1) / (16 * MT)), (unsigned)z);
    if (grid.x == 0 || grid.y == 0) return LLMK_OK;
    kern<<<grid, MD_THREADS, lds_bytes, stream>>>(q);
    LLMK_CHECK_LAUNCH(name);
    if (split) {
        const int64_t mn = (int64_t)p.M * p.N;
        const unsigned blocks = (unsigned)cdiv64(cdiv64(mn, 4), 256);
        if constexpr (KIND == K_I8_ROWCOL) {
            const int32_t* part = (const int32_t*)p.partial;
            if (p.c_dtype == LLMK_BF16) splitk_sum_rowcol_kernel<LLMK_BF16><<<blocks, 256, 0, stream>>>(part, p, mn, z);
            else if (p.c_dtype == LLMK_F16) splitk_sum_rowcol_kernel<LLMK_F16><<<blocks, 256, 0, stream>>>(part, p, mn, z);
            else splitk_sum_rowcol_kernel<LLMK_F32><<<blocks, 256, 0, stream>>>(part, p, mn, z);
        } else {
            if (p.c_dtype == LLMK_BF16) splitk_sum_kernel<LLMK_BF16><<<blocks, 256, 0, stream>>>(p.partial, p.c, mn, z);
            else if (p.c_dtype == LLMK_F16) splitk_sum_kernel<LLMK_F16><<<blocks, 256, 0, stream>>>(p.partial, p.c, mn, z);
            else splitk_sum_kernel<LLMK_F32><<<blocks, 256, 0, stream>>>(p.partial, p.c, mn, z);
        }
        LLMK_CHECK_LAUNCH(name);
    }
    return LLMK_OK;
}

}  // namespace llmk
